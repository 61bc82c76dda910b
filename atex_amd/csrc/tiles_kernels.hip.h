// LayerNorm over rows too long to keep in registers (more than 4096 / 2048 vectors,
// forward / backward): the [N, D] problem is cut into 2-D tiles of R rows x CW columns,
// CW = kTileThreads * kTileVpt * V, one workgroup per tile.  A thread owns the same
// kTileVpt column vectors for every row of its tile, so gamma / beta and the dgamma / dbeta
// accumulators of those columns stay in registers while the rows stream through: x and dy
// are read once per stage, the per-column parameters once per tile.
//
// Replaces the reference's multi-block fallbacks (fused_layer_norm_op.cu:523-561, 573-633,
// 635-719) and its separate dgamma / dbeta pass (:742-803) for such rows.
//
// Rows may have any length and any element alignment: full vectors use 16-byte accesses
// (the hardware takes them at element alignment), and the one partial vector at the end of
// a row whose length is not a multiple of V is handled, element by element, by the single
// thread that owns it ("tail slot"), outside the vector code of everybody else.
//
// The backward sums kernel also comes with narrower tiles (1 or 2 vectors per thread): with
// few column tiles a launch needs many row slabs to fill the chip, and every slab costs a
// partial dgamma / dbeta row of 2 * D floats; narrower tiles mean fewer slabs.
//
// Stages:  forward   split_fwd_stats -> merge_row_stats -> tile_fwd_apply
//          backward  tile_bwd_sums -> merge_row_sums -> tile_bwd_apply [-> col_reduce]
#pragma once

#include "norm_common.hip.h"

namespace atexn {

constexpr int kTileThreads = 256;
constexpr int kTileVpt = 4;
constexpr int kTileRowGroup = 64;  // rows whose wave sums are staged in LDS between barriers

template <int V, int VPT = kTileVpt>
struct TileGeom {
  int64_t r0, r1;            // rows of the tile
  int64_t col[VPT];          // first column of each owned vector (clamped into the row)
  bool full[VPT];            // the vector lies wholly inside the row
  bool has_tail;             // this thread owns the row's partial last vector
  int64_t tail_col;
  int tail_cnt;
};

// Tiles are indexed (blockIdx.x = column tile, blockIdx.y = row slab).
template <int V, int VPT = kTileVpt>
__device__ __forceinline__ TileGeom<V, VPT> tile_geom(int64_t n_rows, int64_t D, int64_t R) {
  TileGeom<V, VPT> g;
  const int64_t CW = static_cast<int64_t>(kTileThreads) * VPT * V;
  const int64_t c0 = static_cast<int64_t>(blockIdx.x) * CW;
  g.r0 = static_cast<int64_t>(blockIdx.y) * R;
  g.r1 = g.r0 + R < n_rows ? g.r0 + R : n_rows;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int64_t c = c0 + (static_cast<int64_t>(threadIdx.x) + k * kTileThreads) * V;
    g.full[k] = c + V <= D;
    // vectors outside the row read (and ignore) the row's last full vector position
    g.col[k] = g.full[k] ? c : (D >= V ? D - V : 0);
  }
  const int rem = static_cast<int>(D % V);
  const int64_t jt = D / V;  // index of the partial vector among the row's vectors
  g.tail_cnt = rem;
  g.tail_col = jt * V;
  g.has_tail = rem != 0 && jt / (kTileThreads * VPT) == blockIdx.x &&
               jt % kTileThreads == threadIdx.x;
  return g;
}

template <typename T, int V>
__device__ __forceinline__ void unpack(const Pack<T, V>& p, float (&f)[V]) {
#pragma unroll
  for (int i = 0; i < V; ++i) f[i] = to_f32(p.v[i]);
}

// ------------------------------------------------------------ per-row merges (one wave per row)
// mean / inv_std of each row from the S per-chunk (mean, m2) pairs of split_fwd_stats; the
// element count of a chunk follows from the geometry.
template <int RPB>  // rows (= waves) per block
__global__ void __launch_bounds__(RPB * kWave)
merge_row_stats(const float2* __restrict__ stats, float* __restrict__ mean_out,
                float* __restrict__ rstd_out, int64_t n_rows, int64_t D, int S, int64_t chunk,
                float eps) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * RPB + threadIdx.x / kWave;
  if (row >= n_rows) return;
  Wf w{0.f, 0.f, 0.f};
  for (int s = lane; s < S; s += kWave) {
    const float2 t = stats[row * S + s];
    const int64_t beg = static_cast<int64_t>(s) * chunk;
    Wf o{t.x, t.y, static_cast<float>(beg + chunk <= D ? chunk : D - beg)};
    w = wf_merge(w, o);
  }
  w = group_wf<kWave>(w);
  if (lane == 0) {
    mean_out[row] = w.mean;
    rstd_out[row] = rsqrtf(w.m2 / static_cast<float>(D) + eps);
  }
}

// rowsum[row] = (sum g, sum g * xh) over the CT column tiles of tile_bwd_sums.
template <int RPB>
__global__ void __launch_bounds__(RPB * kWave)
merge_row_sums(const float2* __restrict__ sums, float2* __restrict__ rowsum, int64_t n_rows,
               int CT) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = static_cast<int64_t>(blockIdx.x) * RPB + threadIdx.x / kWave;
  if (row >= n_rows) return;
  float a = 0.f, b = 0.f;
  const float2* p = sums + row * CT;
  constexpr int B = 4;
  batched_for<B>(
      lane, CT, kWave,
      [&](int64_t c, int64_t step) {
        float2 t[B];
#pragma unroll
        for (int u = 0; u < B; ++u) t[u] = p[c + u * step];
#pragma unroll
        for (int u = 0; u < B; ++u) {
          a += t[u].x;
          b += t[u].y;
        }
      },
      [&](int64_t c) {
        const float2 t = p[c];
        a += t.x;
        b += t.y;
      });
  a = group_sum<kWave>(a);
  b = group_sum<kWave>(b);
  if (lane == 0) rowsum[row] = make_float2(a, b);
}

// ------------------------------------------------------------------------ forward, stage 3
// y = (x - mean[row]) * rstd[row] * gamma + beta over one tile.  y may alias x (every
// element is read by the thread that writes it, before it writes it).
template <typename T, int V>
__global__ void __launch_bounds__(kTileThreads)
tile_fwd_apply(const T* x, const float* __restrict__ gamma, const float* __restrict__ beta,
               const float* __restrict__ mean_in, const float* __restrict__ rstd_in, T* y,
               int64_t n_rows, int64_t D, int64_t R, int rev) {
  const TileGeom<V> g = tile_geom<V>(n_rows, D, R);
  float gm[kTileVpt][V], bt[kTileVpt][V];
#pragma unroll
  for (int k = 0; k < kTileVpt; ++k) {
    load_f32<V>(gamma + g.col[k], gm[k]);
    load_f32<V>(beta + g.col[k], bt[k]);
  }
  float tg[V], tb[V];
  if (g.has_tail) {
    load_f32_n<V>(gamma + g.tail_col, tg, g.tail_cnt);
    load_f32_n<V>(beta + g.tail_col, tb, g.tail_cnt);
  }
  const int64_t n = g.r1 - g.r0;
  for (int64_t i = 0; i < n; ++i) {
    // rev: start from the slab's last row, the one the statistics pass read last
    const int64_t row = rev ? g.r1 - 1 - i : g.r0 + i;
    const T* xr = x + row * D;
    T* yr = y + row * D;
    Pack<T, V> pk[kTileVpt];
#pragma unroll
    for (int k = 0; k < kTileVpt; ++k) pk[k] = load_pack_last<T, V>(xr + g.col[k]);
    const float mean = mean_in[row], rstd = rstd_in[row];
#pragma unroll
    for (int k = 0; k < kTileVpt; ++k) {
      float f[V];
      unpack<T, V>(pk[k], f);
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) o.v[e] = from_f32<T>((f[e] - mean) * rstd * gm[k][e] + bt[k][e]);
      if (g.full[k]) store_pack<T, V>(yr + g.col[k], o);
    }
    if (g.has_tail) {
      const Pack<T, V> tp = load_pack_n<T, V>(xr + g.tail_col, g.tail_cnt);
      float f[V];
      unpack<T, V>(tp, f);
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) o.v[e] = from_f32<T>((f[e] - mean) * rstd * tg[e] + tb[e]);
      store_pack_n<T, V>(yr + g.tail_col, o, g.tail_cnt);
    }
  }
}

// ----------------------------------------------------------------------- backward, stage 1
// Per row of the tile: (sum g, sum g * xh) over the tile's columns, g = dy * gamma, into
// sums[row * CT + tile]; per column of the tile: sum over the tile's rows of dy * xh and of
// dy, into out_g / out_b (+ slab * slab_stride): the final dgamma / dbeta when there is one
// row slab, the partial rows of col_reduce otherwise.
template <typename T, int V, int VPT>
__global__ void __launch_bounds__(kTileThreads)
tile_bwd_sums(const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ gamma,
              const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
              float2* __restrict__ sums, float* __restrict__ out_g, float* __restrict__ out_b,
              int64_t slab_stride, int64_t n_rows, int64_t D, int64_t R) {
  constexpr int NW = kTileThreads / kWave;
  __shared__ float2 wsum[kTileRowGroup][NW];
  const TileGeom<V, VPT> g = tile_geom<V, VPT>(n_rows, D, R);
  const int CT = gridDim.x;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  float gm[VPT][V], ag[VPT][V], ab[VPT][V];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    load_f32<V>(gamma + g.col[k], gm[k]);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      ag[k][e] = 0.f;
      ab[k][e] = 0.f;
      if (!g.full[k]) gm[k][e] = 0.f;  // a vector outside the row contributes nothing
    }
  }
  float tg[V], tag[V], tab[V];
#pragma unroll
  for (int e = 0; e < V; ++e) tg[e] = tag[e] = tab[e] = 0.f;
  if (g.has_tail) load_f32_n<V>(gamma + g.tail_col, tg, g.tail_cnt);

  for (int64_t base = g.r0; base < g.r1; base += kTileRowGroup) {
    const int64_t end = base + kTileRowGroup < g.r1 ? base + kTileRowGroup : g.r1;
    for (int64_t row = base; row < end; ++row) {
      const T* xr = x + row * D;
      const T* dr = dy + row * D;
      Pack<T, V> px[VPT], pd[VPT];
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        px[k] = load_pack<T, V>(xr + g.col[k]);
        pd[k] = load_pack<T, V>(dr + g.col[k]);
      }
      const float mean = mean_in[row], rstd = rstd_in[row];
      float s1 = 0.f, s2 = 0.f;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        float fx[V], fd[V];
        unpack<T, V>(px[k], fx);
        unpack<T, V>(pd[k], fd);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh = (fx[e] - mean) * rstd;
          const float d = g.full[k] ? fd[e] : 0.f;
          const float gv = d * gm[k][e];
          s1 += gv;
          s2 += gv * xh;
          ag[k][e] += d * xh;
          ab[k][e] += d;
        }
      }
      if (g.has_tail) {
        // elements past the row's end read as dy = 0 and add nothing
        const Pack<T, V> tx = load_pack_n<T, V>(xr + g.tail_col, g.tail_cnt);
        const Pack<T, V> td = load_pack_n<T, V>(dr + g.tail_col, g.tail_cnt);
        float fx[V], fd[V];
        unpack<T, V>(tx, fx);
        unpack<T, V>(td, fd);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          const float xh = (fx[e] - mean) * rstd;
          const float gv = fd[e] * tg[e];
          s1 += gv;
          s2 += gv * xh;
          tag[e] += fd[e] * xh;
          tab[e] += fd[e];
        }
      }
      s1 = group_sum<kWave>(s1);
      s2 = group_sum<kWave>(s2);
      if (lane == 0) wsum[row - base][wave] = make_float2(s1, s2);
    }
    __syncthreads();
    const int64_t row = base + threadIdx.x;
    if (row < end) {
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        a += wsum[threadIdx.x][w].x;
        b += wsum[threadIdx.x][w].y;
      }
      sums[row * CT + blockIdx.x] = make_float2(a, b);
    }
    __syncthreads();
  }

  float* og = out_g + static_cast<int64_t>(blockIdx.y) * slab_stride;
  float* ob = out_b + static_cast<int64_t>(blockIdx.y) * slab_stride;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    if (g.full[k]) {
      store_f32<V>(og + g.col[k], ag[k]);
      store_f32<V>(ob + g.col[k], ab[k]);
    }
  }
  if (g.has_tail) {
    store_f32_n<V>(og + g.tail_col, tag, g.tail_cnt);
    store_f32_n<V>(ob + g.tail_col, tab, g.tail_cnt);
  }
}

// ----------------------------------------------------------------------- backward, stage 3
// dx = rstd * (g - s1 / D - xh * s2 / D), (s1, s2) = rowsum[row].  dx may alias dy.
template <typename T, int V>
__global__ void __launch_bounds__(kTileThreads)
tile_bwd_apply(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
               const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
               const float2* __restrict__ rowsum, T* dx, int64_t n_rows, int64_t D, int64_t R,
               int rev) {
  const TileGeom<V> g = tile_geom<V>(n_rows, D, R);
  const float inv_d = 1.0f / static_cast<float>(D);
  float gm[kTileVpt][V];
#pragma unroll
  for (int k = 0; k < kTileVpt; ++k) load_f32<V>(gamma + g.col[k], gm[k]);
  float tg[V];
  if (g.has_tail) load_f32_n<V>(gamma + g.tail_col, tg, g.tail_cnt);
  const int64_t n = g.r1 - g.r0;
  for (int64_t i = 0; i < n; ++i) {
    const int64_t row = rev ? g.r1 - 1 - i : g.r0 + i;
    const T* xr = x + row * D;
    const T* dr = dy + row * D;
    T* outr = dx + row * D;
    Pack<T, V> px[kTileVpt], pd[kTileVpt];
#pragma unroll
    for (int k = 0; k < kTileVpt; ++k) {
      px[k] = load_pack_last<T, V>(xr + g.col[k]);
      pd[k] = load_pack_last<T, V>(dr + g.col[k]);
    }
    const float mean = mean_in[row], rstd = rstd_in[row];
    const float2 rs = rowsum[row];
    // dx = rstd * g + cb * (x - mean) + cc
    const float cb = -rstd * rstd * rs.y * inv_d;
    const float cc = -rstd * rs.x * inv_d;
#pragma unroll
    for (int k = 0; k < kTileVpt; ++k) {
      float fx[V], fd[V];
      unpack<T, V>(px[k], fx);
      unpack<T, V>(pd[k], fd);
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        o.v[e] = from_f32<T>(rstd * (fd[e] * gm[k][e]) + (cb * (fx[e] - mean) + cc));
      }
      if (g.full[k]) store_pack<T, V>(outr + g.col[k], o);
    }
    if (g.has_tail) {
      const Pack<T, V> tx = load_pack_n<T, V>(xr + g.tail_col, g.tail_cnt);
      const Pack<T, V> td = load_pack_n<T, V>(dr + g.tail_col, g.tail_cnt);
      float fx[V], fd[V];
      unpack<T, V>(tx, fx);
      unpack<T, V>(td, fd);
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        o.v[e] = from_f32<T>(rstd * (fd[e] * tg[e]) + (cb * (fx[e] - mean) + cc));
      }
      store_pack_n<T, V>(outr + g.tail_col, o, g.tail_cnt);
    }
  }
}

}  // namespace atexn
