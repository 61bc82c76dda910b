// Kernels for channels-last InstanceNorm, x viewed as [N, D, C] (D = product of the
// spatial dims).  They replace the reference's channel-last ladder
//   forward   fused_instance_norm_op.cu:23-101 (ToTemp / TempToOut), :774-818 (update),
//             :1066-1165 (smem variant)
//   backward  fused_instance_norm_op.cu:666-730, :103-146, :732-772
// The reference maps one channel to a lane (2-byte loads for fp16, a grid of
// DivUp(C,32) x ppr x N blocks).  Here a lane owns one 128-bit vector of V adjacent
// channels, TPP lanes cover a pixel, and a block of 256 threads sweeps 256 / TPP pixels
// per step, so every wave-load is a contiguous 1 KiB.  The spatial extent of one
// instance is cut into S slabs, one block per (instance, slab, channel tile), two launches:
//   stage 1  per-slab per-channel partials (forward: mean and sum of squared deviations;
//            backward: the two sums) -> workspace
//   stage 2  every block first merges the S partials of its instance and channel tile
//            (a few KiB from L2) into LDS, then applies; no separate finalize launch.
// Small slabs stay in registers between their (single, fully overlapped) batch of loads
// and their use.
#pragma once

#include <type_traits>

#include "norm_common.hip.h"

namespace atexn {

constexpr int kClThreads = 256;
constexpr int kClMaxTileChannels = 2048;  // 256 lanes x 8 channels

// Thread geometry.  TPP: threads per pixel (power of two, <= 256; tpp_shift = log2 TPP).
// The grid is (instances, slabs, channel tiles): the instance is the fastest-varying block
// coordinate so that, with workgroups dealt round-robin to the XCDs, the slabs of one
// instance share an XCD and its L2 whenever N is a multiple of the XCD count.
struct ClGeom {
  int64_t n;       // instance
  int s;           // slab
  int ct;          // channel tile
  int cvi;         // channel-vector index of this thread
  int coff;        // first channel of the thread's vector: cvi * V, except that the last
                   //   vector of a C that is not a multiple of V starts at C - V (it overlaps
                   //   its neighbour) and owns only its elements lo .. V-1
  int lo;
  int lo_out;      // first element of the vector that the thread writes to y / dx: the elements
                   //   lo_out .. lo - 1 of an overlapping last vector belong to the neighbour,
                   //   which computes the same bits for them from the same inputs and constants,
                   //   so both may store the full vector (lo_out = 0); only where the vector
                   //   reaches into the previous channel tile, whose constants this workgroup
                   //   does not have, or where the neighbour sits in another wave (in-place
                   //   calls: that wave may already have overwritten x), the thread keeps to
                   //   its own elements (lo_out = lo)
  int slot;        // pixel slot inside the block
  int ppb;         // pixel slots per block
  bool ch_ok;      // channel vector inside C
  int64_t p0, p1;  // pixel range of the slab
  int slab_n;      // p1 - p0 (resident slabs only: they have at most 16 * 256 pixels)
};

// Geometry of the thread for instance n, slab s, channel tile ct.
template <bool RG>
__device__ __forceinline__ ClGeom cl_geom_at(int64_t n, int s, int ct, int tpp_shift, int CV, int C, int V,
                                             int64_t D, int64_t slab_len) {
  ClGeom g;
  g.n = n;
  g.s = s;
  g.ct = ct;
  const int t = static_cast<int>(threadIdx.x);
  g.cvi = (g.ct << tpp_shift) | (t & ((1 << tpp_shift) - 1));
  g.slot = t >> tpp_shift;
  g.ppb = kClThreads >> tpp_shift;
  g.ch_ok = g.cvi < CV;
  const int nominal = (g.ch_ok ? g.cvi : CV - 1) * V;
  if constexpr (RG) {  // C is not a multiple of V (and C >= V)
    g.coff = nominal + V <= C ? nominal : C - V;
    g.lo = g.ch_ok ? nominal - g.coff : 0;
    g.lo_out = g.coff >= (g.ct << tpp_shift) * V && (t & (kWave - 1)) != 0 ? 0 : g.lo;
  } else {
    g.coff = nominal;
    g.lo = 0;
    g.lo_out = 0;
  }
  g.p0 = static_cast<int64_t>(g.s) * slab_len;
  g.p1 = g.p0 + slab_len < D ? g.p0 + slab_len : D;
  g.slab_n = static_cast<int>(g.p1 - g.p0 < (1 << 20) ? g.p1 - g.p0 : (1 << 20));
  return g;
}
// The same for a launch whose grid is (N, S, channel tiles).
template <bool RG>
__device__ __forceinline__ ClGeom cl_geom(int tpp_shift, int CV, int C, int V, int64_t D,
                                          int64_t slab_len) {
  return cl_geom_at<RG>(blockIdx.x, static_cast<int>(blockIdx.y), static_cast<int>(blockIdx.z), tpp_shift, CV, C,
                        V, D, slab_len);
}

// v + v of the lane whose id differs in bit M: VALU cross-lane forms where the ISA has
// one (quad permutes, row rotate by 8, the 16- and 32-lane swaps), the LDS crossbar
// otherwise.  Symmetric, so both partners end with the same bits.
template <int M>
__device__ __forceinline__ float xor_add(float v) {
  if constexpr (M == 1) return v + dpp_read<kDppQuadXor1>(v);
  if constexpr (M == 2) return v + dpp_read<kDppQuadXor2>(v);
  if constexpr (M == 4) return v + lane_xor(v, 4);
  if constexpr (M == 8) return v + dpp_read<0x128>(v);  // row_ror:8
  if constexpr (M == 16) return swap_add<16>(v);
  if constexpr (M == 32) return swap_add<32>(v);
}

// Sum over the lanes of a wave that own the same channels (lane ids equal modulo TPP0),
// for K values at once; TPP0 is a compile-time power of two <= 32.
template <int K, int TPP0>
__device__ __forceinline__ void strided_wave_sum(float (&v)[K]) {
#pragma unroll
  for (int i = 0; i < K; ++i) {
    float t = v[i];
    if constexpr (TPP0 <= 1) t = xor_add<1>(t);
    if constexpr (TPP0 <= 2) t = xor_add<2>(t);
    if constexpr (TPP0 <= 4) t = xor_add<4>(t);
    if constexpr (TPP0 <= 8) t = xor_add<8>(t);
    if constexpr (TPP0 <= 16) t = xor_add<16>(t);
    if constexpr (TPP0 <= 32) t = xor_add<32>(t);
    v[i] = t;
  }
}

// Sum K per-thread values over all threads of the block that own the same channels
// (same threadIdx.x % TPP).  Every such thread ends with the same total, added in a
// fixed order.  lds: K * 256 floats; the caller must __syncthreads() before reusing it.
template <int K>
__device__ __forceinline__ void cl_block_sum(float (&v)[K], float* lds, int TPP) {
  switch (TPP) {  // one uniform branch; threads per pixel is a power of two
    case 1: strided_wave_sum<K, 1>(v); break;
    case 2: strided_wave_sum<K, 2>(v); break;
    case 4: strided_wave_sum<K, 4>(v); break;
    case 8: strided_wave_sum<K, 8>(v); break;
    case 16: strided_wave_sum<K, 16>(v); break;
    case 32: strided_wave_sum<K, 32>(v); break;
    default: break;  // 64 and up: a wave holds every channel vector at most once
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  constexpr int NW = kClThreads / kWave;
  if (TPP == kClThreads) return;  // every thread owns its channels alone
#pragma unroll
  for (int i = 0; i < K; ++i) lds[(i * NW + wave) * kWave + lane] = v[i];
  __syncthreads();
  if (TPP <= kWave) {  // every wave holds the same channel vectors: sum all NW of them
#pragma unroll
    for (int i = 0; i < K; ++i) {
      float s = lds[(i * NW) * kWave + lane];
#pragma unroll
      for (int w = 1; w < NW; ++w) s += lds[(i * NW + w) * kWave + lane];
      v[i] = s;
    }
  } else {  // TPP == 128: waves w and w + 2 share channel vectors
#pragma unroll
    for (int i = 0; i < K; ++i) {
      v[i] = lds[(i * NW + (wave & 1)) * kWave + lane] + lds[(i * NW + (wave & 1) + 2) * kWave + lane];
    }
  }
}

// How the threads of a block split the fold over S partial rows for the channels of a
// tile of `cap` channels (cap = TPP * V, a power of two): P adjacent lanes per channel
// when the tile has at most 256 channels, else one lane per channel and several sweeps.
// Slab partials per lane up to which a fold keeps all of them in registers: kClFoldRegs, or
// twice that by a second variant of the code.
constexpr int kClFoldRegs = 16;

// base[at], or 0 when the position is not the lane's (the load itself is unconditional and
// `at` then names valid memory).
__device__ __forceinline__ float q_or_zero(const float* base, unsigned at, bool mine) {
  const float v = base[at];
  return mine ? v : 0.f;
}

struct FoldMap {
  int P;       // lanes per channel (power of two, <= 64)
  int sweeps;  // passes over the tile when it has more channels than threads
};
__device__ __forceinline__ FoldMap fold_map(int cap) {
  FoldMap m;
  if (cap >= kClThreads) {
    m.P = 1;
    m.sweeps = cap / kClThreads;
  } else {
    m.P = kClThreads / cap < kWave ? kClThreads / cap : kWave;
    m.sweeps = 1;
  }
  return m;
}

template <int B, typename Full, typename Tail>
__device__ __forceinline__ void cl_for_pixels(const ClGeom& g, Full&& full, Tail&& tail) {
  batched_for<B>(g.p0 + g.slot, g.p1, g.ppb, full, tail);
}

// Resident slabs (U > 0): a thread holds the U pixels of its slot as raw vectors.  Loads
// are unconditional so that they are all in flight at once: a lane whose pixel or channel
// vector lies outside the slab reads the slab's first pixel / the last channel vector
// instead (always valid memory) and is masked out of the arithmetic.
// Positions inside a slab are 32-bit element offsets from the slab's first pixel (`slab`, the
// same address for the whole workgroup): a resident slab has at most 4096 pixels and the
// planner keeps 4096 * C * sizeof(T) below 2^31, so no thread carries 64-bit addresses for its
// U pixels through the kernel.
__device__ __forceinline__ unsigned cl_slab_offset(const ClGeom& g, int C, int u) {
  return static_cast<unsigned>(g.slot + u * g.ppb) * static_cast<unsigned>(C) + static_cast<unsigned>(g.coff);
}

// A copy of the geometry whose per-thread fields the compiler treats as new values: a load
// through it, on a path that is seldom taken, computes its addresses there instead of keeping
// those of the kernel's first load alive (sixteen registers) all the way through the common path.
__device__ __forceinline__ ClGeom cl_geom_again(const ClGeom& g) {
  ClGeom h = g;
  asm volatile("" : "+v"(h.slot), "+v"(h.coff));
  return h;
}

// FULL: the host has checked that every slab of the launch has exactly U pixels per slot and that
// every channel tile is complete, so every lane's every vector is valid: ok[] are compile-time
// constants and the masks they feed disappear from the arithmetic (a third of the instructions
// of the statistics, which run after the loads and are what the stage-1 kernels wait on).
template <typename T, int V, int U, bool LAST = false, bool FULL = false>
__device__ __forceinline__ void cl_load_slab(const T* slab, const ClGeom& g, int C,
                                             Pack<T, V> (&raw)[U], bool (&ok)[U]) {
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const bool inside = FULL || g.slot + u * g.ppb < g.slab_n;
    ok[u] = FULL || (g.ch_ok && inside);
    const T* src = slab + (inside ? cl_slab_offset(g, C, u) : static_cast<unsigned>(g.coff));
    raw[u] = LAST ? load_pack_last<T, V>(src) : load_pack<T, V>(src);
  }
}

// ------------------------------------------------------- building blocks of the stages
// Statistics of a register-resident slab: an exact two-pass over the registers (block-wide
// sum -> slab mean, block-wide sum of squared deviations from it).  lds: V * 256 floats.
template <typename T, int V, int U>
__device__ __forceinline__ void cl_resident_stats(const Pack<T, V> (&raw)[U], const bool (&ok)[U],
                                                  float inv_n, int TPP, float* lds,
                                                  float (&mean)[V], float (&m2)[V]) {
  const float one = mix_one();
#pragma unroll
  for (int i = 0; i < V; ++i) mean[i] = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) mean[i] = ok[u] ? add_f32<T>(mean[i], raw[u].v[i], one) : mean[i];
  }
  cl_block_sum<V>(mean, lds, TPP);
#pragma unroll
  for (int i = 0; i < V; ++i) {
    mean[i] *= inv_n;
    m2[i] = 0.f;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float d = ok[u] ? sub_f32<T>(raw[u].v[i], mean[i], one) : 0.f;
      m2[i] = __builtin_fmaf(d, d, m2[i]);
    }
  }
  __syncthreads();  // the first sum's LDS reads are done
  cl_block_sum<V>(m2, lds, TPP);
}

// Combination of the S slab statistics pstat[(n * S + s)][2][C] of every channel of the block's
// tile (and, from the block of slab 0, into the op's outputs), in two
// sweeps over the partials (a few KiB, cache-resident):
//     mean = sum_s n_s mean_s / D,      m2 = sum_s [ m2_s + n_s (mean_s - mean)^2 ]
// which is Chan's merge (norm_util.h:190-210) of all slabs at once: every term of m2 is
// non-negative, nothing cancels, and there is no division or dependent chain per slab.  Each of
// the fm.P lanes of a channel takes every P-th slab in order, then the lanes add pairwise
// (commutative, so every workgroup of the instance gets the same bits).  The counts follow from
// cnt_len (the slab length; after cl_merge_stats S == 1 and cnt_len == D).  The lane that ends
// up with a channel's statistics also fetched its gamma / beta (issued with the partials, one
// round trip) and leaves the constants of y = (x - sm_mean) * sm_sc + sm_bt in LDS, so that no
// thread of the apply phase loads anything but x.  The caller synchronises the block before it
// reads them.
template <bool WIDE>
__device__ __forceinline__ void cl_fold_stats(const float* pstat, const ClGeom& g, int S,
                                              int64_t cnt_len, int64_t D, int C, int cap,
                                              float eps, const float* __restrict__ gamma,
                                              const float* __restrict__ beta, float* sm_mean,
                                              float* sm_sc, float* sm_bt,
                                              float* __restrict__ mean_out,
                                              float* __restrict__ rstd_out) {
  // (the kernels that share this fold must produce the same bits from the same partials:
  // which multiply-adds get fused is not left to the compiler's choice per kernel)
#pragma clang fp contract(off)
  const FoldMap fm = fold_map(cap);
  const float inv_d = 1.0f / static_cast<float>(D);
  const float n_full = static_cast<float>(cnt_len);
  const float n_last = static_cast<float>(D - static_cast<int64_t>(S - 1) * cnt_len);
  const int c_base = g.ct * cap;
  // The partials of the instance: one address for the whole workgroup; positions inside are
  // 32-bit (the planner keeps 2 * S * C below 2^32).
  const float* q = pstat + ((g.n * S) * 2) * C;
  const unsigned uC = static_cast<unsigned>(C), uS = static_cast<unsigned>(S);
  const unsigned P = static_cast<unsigned>(fm.P);
  for (int sweep = 0; sweep < fm.sweeps; ++sweep) {
    const int cl = sweep * kClThreads + static_cast<int>(threadIdx.x) / fm.P;  // channel in tile
    const unsigned sub = static_cast<unsigned>(threadIdx.x) % P;
    const int c = c_base + cl;
    const bool in = cl < cap && c < C;
    const unsigned cc = in ? static_cast<unsigned>(c) : 0u;
    float gm = 0.f, bt = 0.f;
    if (sub == 0 && in) {
      gm = gamma[c];
      bt = beta[c];
    }
    constexpr int B = 16;
    float s1 = 0.f, m2 = 0.f, mean;
    // few slabs per lane (at most R): all of a lane's (mean, m2) pairs are loaded at once, one
    // memory round trip for both sweeps (a lane without a slab in a position reads slab 0 and
    // weighs it 0); same order of additions as the general path below
    auto from_registers = [&](auto rc) {
      constexpr int R = decltype(rc)::value;
      float tm[R], tq[R];
      auto weight = [&](int u) {
        const unsigned sl = sub + u * P;
        return !(in && sl < uS) ? 0.f : (sl == uS - 1 ? n_last : n_full);
      };
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const unsigned sl = sub + u * P;
        const unsigned at = in && sl < uS ? sl : 0u;
        tm[u] = q[(at * 2) * uC + cc];
        tq[u] = q[(at * 2 + 1) * uC + cc];
      }
#pragma unroll
      for (int u = 0; u < R; ++u) s1 += tm[u] * weight(u);
      for (int m = 1; m < fm.P; m <<= 1) s1 += lane_xor(s1, m);
      mean = s1 * inv_d;
#pragma unroll
      for (int u = 0; u < R; ++u) {
        const float d = tm[u] - mean;
        const float tn = weight(u);
        m2 += tn == 0.f ? 0.f : tq[u] + tn * (d * d);
      }
    };
    if (uS <= kClFoldRegs * P) {
      from_registers(std::integral_constant<int, kClFoldRegs>{});
    } else if (WIDE && uS <= 2 * kClFoldRegs * P) {
      from_registers(std::integral_constant<int, WIDE ? 2 * kClFoldRegs : 1>{});
    } else {
      if (in) {
        for (unsigned sl = sub; sl < uS; sl += B * P) {
          float tm[B], tn[B];
#pragma unroll
          for (int u = 0; u < B; ++u) {
            const unsigned k = sl + u * P;
            tm[u] = q[((k < uS ? k : 0u) * 2) * uC + cc];
            tn[u] = k >= uS ? 0.f : (k == uS - 1 ? n_last : n_full);
          }
#pragma unroll
          for (int u = 0; u < B; ++u) s1 += tm[u] * tn[u];
        }
      }
      for (int m = 1; m < fm.P; m <<= 1) s1 += lane_xor(s1, m);
      mean = s1 * inv_d;
      if (in) {
        for (unsigned sl = sub; sl < uS; sl += B * P) {
          float tm[B], tq[B], tn[B];
#pragma unroll
          for (int u = 0; u < B; ++u) {
            const unsigned k = sl + u * P;
            const unsigned at = k < uS ? k : 0u;
            tm[u] = q[(at * 2) * uC + cc];
            tq[u] = q[(at * 2 + 1) * uC + cc];
            tn[u] = k >= uS ? 0.f : (k == uS - 1 ? n_last : n_full);
          }
#pragma unroll
          for (int u = 0; u < B; ++u) {
            const float d = tm[u] - mean;
            m2 += tn[u] == 0.f ? 0.f : tq[u] + tn[u] * (d * d);
          }
        }
      }
    }
    for (int m = 1; m < fm.P; m <<= 1) m2 += lane_xor(m2, m);
    if (sub == 0 && in) {
      const float rs = rsqrtf(__builtin_fmaf(m2, inv_d, eps));
      sm_mean[cl] = mean;
      sm_sc[cl] = gm * rs;
      sm_bt[cl] = bt;
      if (g.s == 0) {
        mean_out[g.n * C + c] = mean;
        rstd_out[g.n * C + c] = rs;
      }
    }
  }
}

// Per-thread constants of the forward apply, read from what cl_fold_stats left in LDS.
template <int V, bool RG>
struct ClFwdCoef {
  float mean[V], sc[V], bt[V];
  __device__ __forceinline__ void load(const ClGeom& g, int tpp_shift, const float* sm_mean,
                                       const float* sm_sc, const float* sm_bt) {
    // channel of element i inside the tile; elements the thread does not own may fall before
    // the tile (their results are never stored)
    const int cl0 = g.coff - ((g.ct << tpp_shift) * V);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int at = RG && cl0 + i < 0 ? 0 : cl0 + i;
      mean[i] = sm_mean[at];
      sc[i] = sm_sc[at];
      bt[i] = sm_bt[at];
    }
  }
  template <typename T>
  __device__ __forceinline__ Pack<T, V> apply(const Pack<T, V>& pk) const {
    Pack<T, V> o;
    const float one = mix_one();
#pragma unroll
    for (int i = 0; i < V; ++i) {
      // subtract the mean first: x * scale - mean * scale would cancel badly when |mean| >> std.
      // (explicit fused multiply-adds: every kernel that applies these constants rounds alike)
      o.v[i] = from_f32<T>(__builtin_fmaf(sub_f32<T>(pk.v[i], mean[i], one), sc[i], bt[i]));
    }
    return o;
  }
};

// Sums of a register-resident slab for the backward: acc[i] = sum dy * xh, acc[V + i] = sum dy
// over the block's pixels, per channel of the thread.  lds: 2 * V * 256 floats.
template <typename T, int V, int U>
__device__ __forceinline__ void cl_resident_sums(const Pack<T, V> (&rx)[U], const Pack<T, V> (&rd)[U],
                                                 const bool (&ok)[U], const float (&mu)[V],
                                                 const float (&rs)[V], int TPP, float* lds,
                                                 float (&acc)[2 * V]) {
  const float one = mix_one();
#pragma unroll
  for (int i = 0; i < 2 * V; ++i) acc[i] = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      // (a masked-out vector leaves the sums as they are; the half operands feed the
      // multiply-adds directly)
      const float xh = sub_f32<T>(rx[u].v[i], mu[i], one) * rs[i];
      acc[i] = ok[u] ? __builtin_fmaf(to_f32(rd[u].v[i]), xh, acc[i]) : acc[i];
      acc[V + i] = ok[u] ? add_f32<T>(acc[V + i], rd[u].v[i], one) : acc[V + i];
    }
  }
  cl_block_sum<2 * V>(acc, lds, TPP);
}

// Backward counterpart of cl_fold_stats: adds up the S slab partials part[(n * S + s)][2][C]
// of the block's instance and channel tile into B = sum dy * xh and A = sum dy, leaves the
// constants of dx = sm_sc * dy + (sm_ca * (x - sm_mu) + sm_cb) in LDS (sc = gamma * r,
// ca = -sc * r * B / D, cb = -sc * A / D; norm_util.h:599-615 in s1 / s2 form; gamma, mean and
// inverse std of a channel are fetched by the lane that folds it, with the partials), and
// produces the block's share of dgamma / dbeta: output o (o < C: dgamma[o], else dbeta[o - C])
// is the sum of one column of all N * S partial rows (fixed order, no atomics); block w of the
// grid takes outputs w, w + #blocks, ...  Ends with a block-wide barrier.  fold_lds: 256 floats.
template <bool WIDE>
__device__ __forceinline__ void cl_fold_sums(const float* part, const ClGeom& g, int64_t N, int S,
                                             int C, int cap, float inv_d,
                                             const float* __restrict__ gamma,
                                             const float* __restrict__ mean_in,
                                             const float* __restrict__ rstd_in, float* sm_mu,
                                             float* sm_sc, float* sm_ca, float* sm_cb,
                                             float (*red_buf)[16], float* fold_lds,
                                             float* __restrict__ dgamma,
                                             float* __restrict__ dbeta, int cw_shift) {
#pragma clang fp contract(off)
  const FoldMap fm = fold_map(cap);
  const int c_base = g.ct * cap;
  const int64_t n_blocks = static_cast<int64_t>(gridDim.x) * gridDim.y * gridDim.z;
  const int64_t w = (static_cast<int64_t>(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
  const int64_t rows = N * S;
  const int64_t W2 = 2 * static_cast<int64_t>(C);  // a partial row: [dgamma terms | dbeta terms]
  // Outputs are dealt to the blocks in chunks of cw = 64, 16, 4 or 1 adjacent columns (the host
  // picks the width that leaves a block the fewest dependent memory round trips,
  // cl_dparam_chunk_shift): the 256 / cw thread rows of a chunk each take every (256 / cw)-th
  // partial row, four at a time.
  const int cw = 1 << cw_shift;
  const int rp = kClThreads >> cw_shift;  // partial rows in flight
  const int cx = static_cast<int>(threadIdx.x) & (cw - 1);
  const int cy = static_cast<int>(threadIdx.x) >> cw_shift;
  const int64_t n_chunks = (W2 + cw - 1) >> cw_shift;
  // At most one chunk per block and at most kEarly partial rows per thread: the chunk's loads
  // are issued here, ahead of the slab fold's, so that both share one memory round trip.
  constexpr int kEarly = 4;
  const bool early = n_chunks <= n_blocks && rows <= static_cast<int64_t>(kEarly) * rp;
  float ev[kEarly];
  if (early) {
    const int64_t col = w * cw + cx;
#pragma unroll
    for (int u = 0; u < kEarly; ++u) {
      const int64_t r = cy + u * rp;
      ev[u] = (col < W2 && r < rows) ? part[r * W2 + col] : 0.f;
    }
  }
  // the partials of the instance: one address for the whole workgroup, 32-bit positions inside
  const float* pr = part + ((g.n * S) * 2) * C;
  const unsigned uC = static_cast<unsigned>(C), uS = static_cast<unsigned>(S);
  const unsigned P = static_cast<unsigned>(fm.P);
  for (int sweep = 0; sweep < fm.sweeps; ++sweep) {
    const int cl = sweep * kClThreads + static_cast<int>(threadIdx.x) / fm.P;
    const unsigned sub = static_cast<unsigned>(threadIdx.x) % P;
    const int c = c_base + cl;
    const bool in = cl < cap && c < C;
    const unsigned cc = in ? static_cast<unsigned>(c) : 0u;
    float gm = 0.f, mu = 0.f, rs = 0.f;
    if (sub == 0 && in) {
      gm = gamma[c];
      mu = mean_in[g.n * C + c];
      rs = rstd_in[g.n * C + c];
    }
    float a = 0.f, b = 0.f;
    // a lane's slabs in batches of 16 or, when that spares a round trip, 32 (the additions are
    // in slab order either way)
    auto in_batches = [&](auto bc) {
      constexpr int B = decltype(bc)::value;
      for (unsigned sl = sub; sl < uS; sl += B * P) {
        float tb[B], ta[B];
#pragma unroll
        for (int u = 0; u < B; ++u) {
          const unsigned k = sl + u * P;
          const unsigned at = k < uS ? k : 0u;
          tb[u] = q_or_zero(pr, (at * 2) * uC + cc, k < uS);
          ta[u] = q_or_zero(pr, (at * 2 + 1) * uC + cc, k < uS);
        }
#pragma unroll
        for (int u = 0; u < B; ++u) {
          b += tb[u];
          a += ta[u];
        }
      }
    };
    if (in) {
      if (!WIDE || uS <= kClFoldRegs * P) {
        in_batches(std::integral_constant<int, kClFoldRegs>{});
      } else {
        in_batches(std::integral_constant<int, WIDE ? 2 * kClFoldRegs : 1>{});
      }
    }
    for (int m = 1; m < fm.P; m <<= 1) {
      a += lane_xor(a, m);
      b += lane_xor(b, m);
    }
    if (sub == 0 && in) {
      const float sc = gm * rs;
      sm_mu[cl] = mu;
      sm_sc[cl] = sc;
      sm_ca[cl] = -(sc * rs) * (b * inv_d);
      sm_cb[cl] = -sc * (a * inv_d);
    }
  }
  if (early) {
    if (w < n_chunks) {  // uniform over the block
      float t[1] = {0.f};
#pragma unroll
      for (int u = 0; u < kEarly; ++u) t[0] += ev[u];
      cl_block_sum<1>(t, fold_lds, cw);
      const int64_t col = w * cw + cx;
      if (cy == 0 && col < W2) (col < C ? dgamma : dbeta)[col < C ? col : col - C] = t[0];
    }
    __syncthreads();
    return;
  }
  if (cw > 1) {
    for (int64_t chunk = w; chunk < n_chunks; chunk += n_blocks) {
      const int64_t col = chunk * cw + cx;
      float t[1] = {0.f};
      if (col < W2) {
        const float* pc = part + col;
        batched_for<4>(
            cy, rows, rp,
            [&](int64_t r, int64_t step) {
              float v[4];
#pragma unroll
              for (int u = 0; u < 4; ++u) v[u] = pc[(r + u * step) * W2];
#pragma unroll
              for (int u = 0; u < 4; ++u) t[0] += v[u];
            },
            [&](int64_t r) { t[0] += pc[r * W2]; });
      }
      cl_block_sum<1>(t, fold_lds, cw);
      if (cy == 0 && col < W2) (col < C ? dgamma : dbeta)[col < C ? col : col - C] = t[0];
      __syncthreads();
    }
  }
  int red_it = 0;
  for (int64_t o = w; cw == 1 && o < W2; o += n_blocks) {
    float t = 0.f;
    const float* pc = part + o;
    batched_for<4>(
        threadIdx.x, rows, kClThreads,
        [&](int64_t r, int64_t step) {
          float v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) v[u] = pc[(r + u * step) * W2];
#pragma unroll
          for (int u = 0; u < 4; ++u) t += v[u];
        },
        [&](int64_t r) { t += pc[r * W2]; });
    t = block_sum1(t, red_buf[red_it & 1], kClThreads / kWave);
    ++red_it;
    if (threadIdx.x == 0) (o < C ? dgamma : dbeta)[o < C ? o : o - C] = t;
  }
  __syncthreads();
}

// Per-thread constants of the backward apply, read from what cl_fold_sums left in LDS.
template <int V, bool RG>
struct ClBwdCoef {
  float mu[V], sc[V], ca[V], cb[V];
  __device__ __forceinline__ void load(const ClGeom& g, int tpp_shift, const float* sm_mu,
                                       const float* sm_sc, const float* sm_ca,
                                       const float* sm_cb) {
    const int cl0 = g.coff - ((g.ct << tpp_shift) * V);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const int at = RG && cl0 + i < 0 ? 0 : cl0 + i;
      mu[i] = sm_mu[at];
      sc[i] = sm_sc[at];
      ca[i] = sm_ca[at];
      cb[i] = sm_cb[at];
    }
  }
  template <typename T>
  __device__ __forceinline__ Pack<T, V> apply(const Pack<T, V>& px, const Pack<T, V>& pd) const {
    Pack<T, V> o;
    const float one = mix_one();
#pragma unroll
    for (int i = 0; i < V; ++i) {
      o.v[i] = from_f32<T>(__builtin_fmaf(sc[i], to_f32(pd.v[i]), __builtin_fmaf(ca[i], sub_f32<T>(px.v[i], mu[i], one), cb[i])));
    }
    return o;
  }
};

// ---------------------------------------------------------------- forward, stage 1
// pstat: [N * S][2][C], the (mean, m2 = sum of squared deviations from that mean) of every
// channel over each slab; the slab's pixel count follows from the geometry.  Nothing is
// accumulated around a pivot or around zero, so the result keeps float32 accuracy whatever
// the data look like (an instance whose border pixels are far from the bulk, a large common
// offset): the counterpart of the reference's Welford pushes (norm_util.h:182-211).
// U > 0: the slab is register-resident (slab_len <= U * pixel slots per block), all its
// loads are in flight at once and the statistics are an exact two-pass over the registers.
// U == 0 streams the slab in batches of 8 pixels per thread: per-thread running (mean, m2)
// by batch-wise Chan updates (wf_lanes_push), combined over the block around the slab mean
// (m2 = sum over threads of m2_t + n_t (mean_t - mean)^2, every term non-negative).
template <typename T, int V, int U, bool RG, bool FULL = false>
__global__ void __launch_bounds__(kClThreads)
cl_fwd_stats(const T* __restrict__ x, float* __restrict__ pstat, int64_t D, int C, int S,
             int tpp_shift, int64_t slab_len) {
  __shared__ float lds[V * kClThreads];
  const int CV = (C + V - 1) / V;
  const int TPP = 1 << tpp_shift;
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, slab_len);
  const T* xn = x + (g.n * D) * C;
  const float inv_n = 1.0f / static_cast<float>(g.p1 - g.p0);
  float mean[V], m2[V];
  if constexpr (U > 0) {
    Pack<T, V> raw[U];
    bool ok[U];
    cl_load_slab<T, V, U, false, FULL>(xn + g.p0 * C, g, C, raw, ok);
    cl_resident_stats<T, V, U>(raw, ok, inv_n, TPP, lds, mean, m2);
  } else {
    WfLanes<V> run;
    wf_lanes_init<V>(run);
    if (g.ch_ok) {
      const T* base = xn + g.coff;
      constexpr int B = 8;
      cl_for_pixels<B>(
          g,
          [&](int64_t p, int64_t step) {
            Pack<T, V> pk[B];
#pragma unroll
            for (int u = 0; u < B; ++u) pk[u] = load_pack<T, V>(base + (p + u * step) * C);
            batch_loaded<T, V, B>(pk);
            float f[B][V];
#pragma unroll
            for (int u = 0; u < B; ++u) {
#pragma unroll
              for (int i = 0; i < V; ++i) f[u][i] = to_f32(pk[u].v[i]);
            }
            wf_lanes_push<V, B>(run, f);
          },
          [&](int64_t p) {
            const Pack<T, V> pk = load_pack<T, V>(base + p * C);
            float f[1][V];
#pragma unroll
            for (int i = 0; i < V; ++i) f[0][i] = to_f32(pk.v[i]);
            wf_lanes_push<V, 1>(run, f);
          });
    }
#pragma unroll
    for (int i = 0; i < V; ++i) mean[i] = run.mean[i] * run.n;
    cl_block_sum<V>(mean, lds, TPP);
#pragma unroll
    for (int i = 0; i < V; ++i) {
      mean[i] *= inv_n;
      const float d = run.mean[i] - mean[i];
      m2[i] = run.m2[i] + run.n * (d * d);
    }
    __syncthreads();  // the first sum's LDS reads are done
    cl_block_sum<V>(m2, lds, TPP);
  }
  if (g.ch_ok && g.slot == 0) {
    const int64_t o = ((g.n * S + g.s) * 2) * C + g.coff;
    store_f32_from<V>(pstat + o, mean, RG ? g.lo : 0);
    store_f32_from<V>(pstat + o + C, m2, RG ? g.lo : 0);
  }
}

// Between the stages, only when an instance has more than kClFoldAbove slabs: combines the S slab
// statistics of every (instance, channel) once, in a fixed order and by the same two sweeps as
// cl_fold_stats, into folded[N][2][C] = (mean, m2 of the whole instance), so that the stage-2
// workgroups need not each do it.  Block = kClMergeChannels channels x (256 / kClMergeChannels)
// slab phases; grid = (channel groups, N).
constexpr int kClMergeChannels = 16;
__global__ void __launch_bounds__(kClThreads)
cl_merge_stats(const float* __restrict__ pstat, float* __restrict__ folded, int64_t D, int C, int S,
               int64_t slab_len) {
  constexpr int PH = kClThreads / kClMergeChannels;
  __shared__ float buf[PH][kClMergeChannels];
  const int cx = threadIdx.x % kClMergeChannels;
  const int ph = threadIdx.x / kClMergeChannels;
  const int c = blockIdx.x * kClMergeChannels + cx;
  const int64_t n = blockIdx.y;
  const bool in = c < C;
  const float n_full = static_cast<float>(slab_len);
  const float n_last = static_cast<float>(D - static_cast<int64_t>(S - 1) * slab_len);
  const float* q = pstat + ((n * S) * 2) * C + (in ? c : 0);
  constexpr int B = 16;
  // the phases' partial sums of a channel, added in phase order
  auto across_phases = [&](float v) {
    buf[ph][cx] = v;
    __syncthreads();
    float r = buf[0][cx];
    for (int k = 1; k < PH; ++k) r += buf[k][cx];
    __syncthreads();
    return r;
  };
  // a phase's slabs ph, ph + PH, ... in batches of B whose loads are all in flight at once; a
  // position past the last slab reads slab 0 and weighs it 0 (no dependent single loads at the
  // end of a phase)
  auto weight = [&](int k) { return k >= S ? 0.f : (k == S - 1 ? n_last : n_full); };
  float s1 = 0.f;
  if (in) {
    for (int sl = ph; sl < S; sl += B * PH) {
      float tm[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const int k = sl + u * PH;
        tm[u] = q[(static_cast<int64_t>(k < S ? k : 0) * 2) * C];
      }
#pragma unroll
      for (int u = 0; u < B; ++u) s1 += tm[u] * weight(sl + u * PH);
    }
  }
  const float mean = across_phases(s1) / static_cast<float>(D);
  float m2 = 0.f;
  if (in) {
    for (int sl = ph; sl < S; sl += B * PH) {
      float tm[B], tq[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const int k = sl + u * PH;
        const int64_t at = k < S ? k : 0;
        tm[u] = q[(at * 2) * C];
        tq[u] = q[(at * 2 + 1) * C];
      }
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const float d = tm[u] - mean;
        const float tn = weight(sl + u * PH);
        m2 += tn == 0.f ? 0.f : tq[u] + tn * (d * d);
      }
    }
  }
  m2 = across_phases(m2);
  if (ph == 0 && in) {
    folded[(n * 2) * C + c] = mean;
    folded[(n * 2 + 1) * C + c] = m2;
  }
}

// ---------------------------------------------------------------- forward, stage 2
// y may alias x: stage 1 has completed (it is an earlier launch on the same stream) and
// every thread reads a vector before it writes the same vector.
template <typename T, int V, int U, bool RG, bool FULL = false>
__global__ void __launch_bounds__(kClThreads, 2)  // two workgroups per CU: a grid of 2 x CUs slabs runs in one round
cl_fwd_apply(const T* x, const float* __restrict__ pstat, const float* __restrict__ gamma,
             const float* __restrict__ beta, T* y, float* __restrict__ mean_out,
             float* __restrict__ rstd_out, int64_t D, int C, int S, int64_t cnt_len,
             int tpp_shift, int64_t slab_len, float eps, int rev) {
  __shared__ float sm_mean[kClMaxTileChannels];
  __shared__ float sm_sc[kClMaxTileChannels];
  __shared__ float sm_bt[kClMaxTileChannels];
  const int CV = (C + V - 1) / V;
  const int cap = (1 << tpp_shift) * V;
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, slab_len);
  // resident slab: its loads are issued first and fly while the partials are merged
  Pack<T, V> raw[U > 0 ? U : 1];
  bool ok[U > 0 ? U : 1];
  if constexpr (U > 0) cl_load_slab<T, V, U, true, FULL>(x + (g.n * D + g.p0) * C, g, C, raw, ok);
  cl_fold_stats<(U > 0)>(pstat, g, S, cnt_len, D, C, cap, eps, gamma, beta, sm_mean, sm_sc, sm_bt, mean_out,
                rstd_out);
  __syncthreads();
  if (g.ch_ok) {
    ClFwdCoef<V, RG> k;
    k.load(g, tpp_shift, sm_mean, sm_sc, sm_bt);
    const int64_t boff = (g.n * D) * C + g.coff;
    auto apply = [&](const Pack<T, V>& pk, int64_t p) {
      store_pack_from<T, V>(y + boff + p * C, k.template apply<T>(pk), RG ? g.lo_out : 0);
    };
    if constexpr (U > 0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (ok[u]) {
          store_pack_from<T, V>(y + (g.n * D + g.p0) * C + cl_slab_offset(g, C, u),
                                k.template apply<T>(raw[u]), RG ? g.lo_out : 0);
        }
      }
    } else {
      constexpr int B = 8;
      // rev: walk the slab from its last pixel (what stage 1 read last is still cached)
      const int64_t flip = g.p0 + g.p1 - 1;
      cl_for_pixels<B>(
          g,
          [&](int64_t p, int64_t step) {
            Pack<T, V> pk[B];
            int64_t q[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
              q[u] = rev ? flip - (p + u * step) : p + u * step;
              pk[u] = load_pack_last<T, V>(x + boff + q[u] * C);
            }
            batch_loaded<T, V, B>(pk);
#pragma unroll
            for (int u = 0; u < B; ++u) apply(pk[u], q[u]);
          },
          [&](int64_t p) {
            const int64_t q = rev ? flip - p : p;
            apply(load_pack_last<T, V>(x + boff + q * C), q);
          });
    }
  }
}

// --------------------------------------------------------------- backward, stage 1
// part[(n * S + s)][0][c] = sum dy * xh, part[...][1][c] = sum dy over the slab.
template <typename T, int V, int U, bool RG, bool FULL = false>
__global__ void __launch_bounds__(kClThreads)
cl_bwd_sums(const T* __restrict__ dy, const T* __restrict__ x,
            const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
            float* __restrict__ part, int64_t D, int C, int S, int tpp_shift,
            int64_t slab_len) {
  __shared__ float lds[2 * V * kClThreads];
  const int CV = (C + V - 1) / V;
  const int TPP = 1 << tpp_shift;
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, slab_len);
  float acc[2 * V];
  Pack<T, V> rx[U > 0 ? U : 1], rd[U > 0 ? U : 1];
  bool ok[U > 0 ? U : 1];
  if constexpr (U > 0) {
    cl_load_slab<T, V, U, false, FULL>(x + (g.n * D + g.p0) * C, g, C, rx, ok);
    cl_load_slab<T, V, U, false, FULL>(dy + (g.n * D + g.p0) * C, g, C, rd, ok);
  }
  float mu[V], rs[V];
#pragma unroll
  for (int i = 0; i < V; ++i) mu[i] = rs[i] = 0.f;
  if (g.ch_ok) {
    load_f32<V>(mean_in + g.n * C + g.coff, mu);
    load_f32<V>(rstd_in + g.n * C + g.coff, rs);
  }
  if constexpr (U > 0) {
    cl_resident_sums<T, V, U>(rx, rd, ok, mu, rs, TPP, lds, acc);
  } else {
#pragma unroll
    for (int i = 0; i < 2 * V; ++i) acc[i] = 0.f;
    auto add = [&](const Pack<T, V>& px, const Pack<T, V>& pd) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = to_f32(pd.v[i]);
        const float xh = (to_f32(px.v[i]) - mu[i]) * rs[i];
        acc[i] += d * xh;
        acc[V + i] += d;
      }
    };
    if (g.ch_ok) {
      const int64_t boff = (g.n * D) * C + g.coff;
      constexpr int B = 4;
      cl_for_pixels<B>(
          g,
          [&](int64_t p, int64_t step) {
            Pack<T, V> px[B], pd[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
              px[u] = load_pack<T, V>(x + boff + (p + u * step) * C);
              pd[u] = load_pack<T, V>(dy + boff + (p + u * step) * C);
            }
            batch_loaded<T, V, B>(px, pd);
#pragma unroll
            for (int u = 0; u < B; ++u) add(px[u], pd[u]);
          },
          [&](int64_t p) {
            add(load_pack<T, V>(x + boff + p * C), load_pack<T, V>(dy + boff + p * C));
          });
    }
    cl_block_sum<2 * V>(acc, lds, TPP);
  }
  if (g.ch_ok && g.slot == 0) {
    float* o = part + ((g.n * S + g.s) * 2) * C + g.coff;
    float t0[V], t1[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      t0[i] = acc[i];
      t1[i] = acc[V + i];
    }
    store_f32_from<V>(o, t0, RG ? g.lo : 0);
    store_f32_from<V>(o + C, t1, RG ? g.lo : 0);
  }
}

// --------------------------------------------------------------- backward, stage 2
// Every block first folds the S slab partials of its instance and channel tile into LDS and
// produces its share of dgamma / dbeta (cl_fold_sums), which spares a third launch, then
// writes dx for its slab.
template <typename T, int V, int U, bool RG, bool FULL = false>
__global__ void __launch_bounds__(kClThreads, 2)  // two workgroups per CU: a grid of 2 x CUs slabs runs in one round
cl_bwd_apply(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
             const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
             const float* __restrict__ part, T* dx, float* __restrict__ dgamma,
             float* __restrict__ dbeta, int64_t N, int64_t D, int C, int S, int tpp_shift,
             int64_t slab_len, int rev, int cw_shift) {
  __shared__ float sm_mu[kClMaxTileChannels];
  __shared__ float sm_sc[kClMaxTileChannels];
  __shared__ float sm_ca[kClMaxTileChannels];
  __shared__ float sm_cb[kClMaxTileChannels];
  __shared__ float red_buf[2][16];
  __shared__ float fold_lds[kClThreads];
  const int CV = (C + V - 1) / V;
  const int cap = (1 << tpp_shift) * V;
  const float inv_d = 1.0f / static_cast<float>(D);
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, slab_len);
  // resident slab: its loads are issued first and fly while the partials are folded
  Pack<T, V> rx[U > 0 ? U : 1], rd[U > 0 ? U : 1];
  bool okp[U > 0 ? U : 1];
  if constexpr (U > 0) {
    cl_load_slab<T, V, U, true, FULL>(x + (g.n * D + g.p0) * C, g, C, rx, okp);
    cl_load_slab<T, V, U, true, FULL>(dy + (g.n * D + g.p0) * C, g, C, rd, okp);
  }
  cl_fold_sums<(U > 0)>(part, g, N, S, C, cap, inv_d, gamma, mean_in, rstd_in, sm_mu, sm_sc, sm_ca, sm_cb,
               red_buf, fold_lds, dgamma, dbeta, cw_shift);
  if (g.ch_ok) {
    ClBwdCoef<V, RG> k;
    k.load(g, tpp_shift, sm_mu, sm_sc, sm_ca, sm_cb);
    const int64_t boff = (g.n * D) * C + g.coff;
    auto apply = [&](const Pack<T, V>& px, const Pack<T, V>& pd, int64_t p) {
      store_pack_from<T, V>(dx + boff + p * C, k.template apply<T>(px, pd), RG ? g.lo_out : 0);
    };
    if constexpr (U > 0) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (okp[u]) {
          store_pack_from<T, V>(dx + (g.n * D + g.p0) * C + cl_slab_offset(g, C, u),
                                k.template apply<T>(rx[u], rd[u]), RG ? g.lo_out : 0);
        }
      }
    } else {
      constexpr int B = 4;
      const int64_t flip = g.p0 + g.p1 - 1;
      cl_for_pixels<B>(
          g,
          [&](int64_t p, int64_t step) {
            Pack<T, V> px[B], pd[B];
            int64_t q[B];
#pragma unroll
            for (int u = 0; u < B; ++u) {
              q[u] = rev ? flip - (p + u * step) : p + u * step;
              px[u] = load_pack_last<T, V>(x + boff + q[u] * C);
              pd[u] = load_pack_last<T, V>(dy + boff + q[u] * C);
            }
            batch_loaded<T, V, B>(px, pd);
#pragma unroll
            for (int u = 0; u < B; ++u) apply(px[u], pd[u], q[u]);
          },
          [&](int64_t p) {
            const int64_t q = rev ? flip - p : p;
            apply(load_pack_last<T, V>(x + boff + q * C), load_pack_last<T, V>(dy + boff + q * C), q);
          });
    }
  }
}

// ------------------------------------------------------------------ single pass
// An instance whose pixels fit the registers of one workgroup per channel tile (D <= U pixel
// slots per thread x pixel slots per block) and a grid that is already wide enough with one
// slab per instance: one launch, x read once.  Counterpart of the reference's single-kernel
// shared-memory variant for channels-last (fused_instance_norm_op.cu:1066-1165), with the
// instance in registers instead of shared memory and an exact two-pass over them (mean, then
// centred squares) instead of Welford merges.  Grid = (N, 1, channel tiles).
// y may alias x: a workgroup loads all of its elements before it stores any.
template <typename T, int V, int U, bool RG>
__global__ void __launch_bounds__(kClThreads)
cl_fwd_fused(const T* x, const float* __restrict__ gamma, const float* __restrict__ beta, T* y,
             float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t D, int C,
             int tpp_shift, float eps) {
  __shared__ float lds[V * kClThreads];
  const int CV = (C + V - 1) / V;
  const int TPP = 1 << tpp_shift;
  const float inv_d = 1.0f / static_cast<float>(D);
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, D);
  Pack<T, V> raw[U];
  bool ok[U];
  cl_load_slab<T, V, U>(x + (g.n * D + g.p0) * C, g, C, raw, ok);
  float gm[V], bt[V];
  load_f32<V>(gamma + g.coff, gm);
  load_f32<V>(beta + g.coff, bt);
  float mean[V];
#pragma unroll
  for (int i = 0; i < V; ++i) mean[i] = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) mean[i] += ok[u] ? to_f32(raw[u].v[i]) : 0.f;
  }
  cl_block_sum<V>(mean, lds, TPP);
  float q[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    mean[i] *= inv_d;
    q[i] = 0.f;
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float d = ok[u] ? to_f32(raw[u].v[i]) - mean[i] : 0.f;
      q[i] += d * d;
    }
  }
  __syncthreads();  // the first sum's LDS reads are done
  cl_block_sum<V>(q, lds, TPP);
  float rs[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    rs[i] = rsqrtf(q[i] * inv_d + eps);
    gm[i] *= rs[i];
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (ok[u]) {
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) o.v[i] = from_f32<T>((to_f32(raw[u].v[i]) - mean[i]) * gm[i] + bt[i]);
      store_pack_from<T, V>(y + (g.n * D) * C + cl_slab_offset(g, C, u), o, RG ? g.lo_out : 0);
    }
  }
  if (g.ch_ok && g.slot == 0) {
    store_f32_from<V>(mean_out + g.n * C + g.coff, mean, RG ? g.lo : 0);
    store_f32_from<V>(rstd_out + g.n * C + g.coff, rs, RG ? g.lo : 0);
  }
}

// Backward counterpart: x and dy of the instance in registers (U <= 8 each).  The per-instance
// sums go to part[n][0][c] = sum dy * xh, part[n][1][c] = sum dy for the column reduction over
// n that follows; with a single instance they are dgamma / dbeta themselves (out0 / out1 then
// point at dgamma / dbeta and `stride` is 0).  dx may alias dy.
template <typename T, int V, int U, bool RG>
__global__ void __launch_bounds__(kClThreads)
cl_bwd_fused(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
             const float* __restrict__ mean_in, const float* __restrict__ rstd_in, T* dx,
             float* __restrict__ out0, float* __restrict__ out1, int64_t stride, int64_t D, int C,
             int tpp_shift) {
  __shared__ float lds[2 * V * kClThreads];
  const int CV = (C + V - 1) / V;
  const int TPP = 1 << tpp_shift;
  const float inv_d = 1.0f / static_cast<float>(D);
  const ClGeom g = cl_geom<RG>(tpp_shift, CV, C, V, D, D);
  Pack<T, V> rx[U], rd[U];
  bool ok[U];
  cl_load_slab<T, V, U, true>(x + (g.n * D + g.p0) * C, g, C, rx, ok);
  cl_load_slab<T, V, U, true>(dy + (g.n * D + g.p0) * C, g, C, rd, ok);
  float mu[V], rs[V], sc[V];
  load_f32<V>(mean_in + g.n * C + g.coff, mu);
  load_f32<V>(rstd_in + g.n * C + g.coff, rs);
  load_f32<V>(gamma + g.coff, sc);
  float acc[2 * V];
#pragma unroll
  for (int i = 0; i < 2 * V; ++i) acc[i] = 0.f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float d = ok[u] ? to_f32(rd[u].v[i]) : 0.f;
      const float h = ok[u] ? (to_f32(rx[u].v[i]) - mu[i]) * rs[i] : 0.f;
      acc[i] += d * h;
      acc[V + i] += d;
    }
  }
  cl_block_sum<2 * V>(acc, lds, TPP);
  float ca[V], cb[V];
#pragma unroll
  for (int i = 0; i < V; ++i) {
    sc[i] *= rs[i];
    ca[i] = -sc[i] * (acc[i] * inv_d);
    cb[i] = -sc[i] * (acc[V + i] * inv_d);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    if (ok[u]) {
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float h = (to_f32(rx[u].v[i]) - mu[i]) * rs[i];
        o.v[i] = from_f32<T>(sc[i] * to_f32(rd[u].v[i]) + (ca[i] * h + cb[i]));
      }
      store_pack_from<T, V>(dx + (g.n * D) * C + cl_slab_offset(g, C, u), o, RG ? g.lo_out : 0);
    }
  }
  if (g.ch_ok && g.slot == 0) {
    float t0[V], t1[V];
#pragma unroll
    for (int i = 0; i < V; ++i) {
      t0[i] = acc[i];
      t1[i] = acc[V + i];
    }
    store_f32_from<V>(out0 + g.n * stride + g.coff, t0, RG ? g.lo : 0);
    store_f32_from<V>(out1 + g.n * stride + g.coff, t1, RG ? g.lo : 0);
  }
}

}  // namespace atexn
