// Kernels for contiguous rows: LayerNorm over [N, D] and channel-first InstanceNorm
// over [N*C, D].  They replace the reference's row ladders
//   forward   fused_layer_norm_op.cu:375-433 (warp/row), :145-193 (block/row, smem),
//             :573-684 (multi-block), fused_instance_norm_op.cu:959-1004, :1167-1194
//   backward  fused_layer_norm_op.cu:21-98, :195-255, :523-561, :635-719, :742-803,
//             fused_instance_norm_op.cu:169-313, :315-366, :594-656
// with two designs:
//   * "resident" kernels: the row lives in VGPRs (TPR threads x VPT 128-bit vectors),
//     is read from HBM exactly once, and its statistics come from an exact two-pass over
//     the registers, each pass one all-reduce across the row's lanes (DPP, LDS across waves);
//   * "split" kernels for channel-first planes that do not fit: a row is cut into S
//     chunks, stage 1 writes per-chunk partials, stage 2 merges them and applies
//     (LayerNorm rows that do not fit go to tiles_kernels.hip.h, many tiny rows to
//     small_kernels.hip.h).
// All of them use 16-byte accesses at element alignment; rows may have any length.
#pragma once

#include "norm_common.hip.h"

namespace atexn {

// Geometry of the thread <-> row mapping.  TPR > 0: TPR (power of two <= 64) lanes per
// row and blockDim.x / TPR rows per block; TPR = 128 or 256 (backward only): a row is held
// by 2 or 4 consecutive waves.  TPR == 0: the whole block owns one row.
template <int TPR>
struct RowMap {
  // bdim: the block size (block_threads())
  __device__ __forceinline__ static int tpr(int bdim) { return TPR ? TPR : bdim; }
  __device__ __forceinline__ static int rows_per_block(int bdim) { return TPR ? bdim / TPR : 1; }
  __device__ __forceinline__ static int lane_in_row() {
    return TPR ? static_cast<int>(threadIdx.x) % TPR : static_cast<int>(threadIdx.x);
  }
  __device__ __forceinline__ static int slot() { return TPR ? static_cast<int>(threadIdx.x) / TPR : 0; }
};

// The LayerNorm backward folds the per-lane dgamma / dbeta sums of the waves of a workgroup
// through LDS (rows_bwd_resident): W floats per LDS access, at most fold_groups_per_pass groups
// of W per lane and pass, so that eight waves stay within kFoldLdsBytes.
constexpr int kFoldLdsBytes = 64 * 1024;
constexpr int kFoldMaxWaves = 8;
template <int V>
constexpr int fold_width() {
  return V % 4 == 0 ? 4 : 1;
}
constexpr int fold_groups_per_pass_rt(int V, int vpt, int tpr) {
  const int w = V % 4 == 0 ? 4 : 1;
  const int lr = tpr < 64 ? tpr : 64;
  const int q = 2 * V * vpt / w;
  const int cap = kFoldLdsBytes / (kFoldMaxWaves * lr * w * 4);
  return q < cap ? q : cap;
}
template <int V, int VPT, int TPR>
constexpr int fold_groups_per_pass() {
  return fold_groups_per_pass_rt(V, VPT, TPR == 0 ? 64 : TPR);
}

// Largest block a resident kernel instantiation is launched with; it fixes the VGPR
// budget the compiler works against (512 VGPRs per SIMD lane / waves per SIMD).
template <int TPR, int VPT>
constexpr int resident_fwd_max_threads() {
  return TPR != 0 ? 256 : (VPT == 2 ? 1024 : (VPT == 4 ? 768 : 512));
}
template <int TPR, bool BWD_COLS, int RB, int VPT>
constexpr int resident_bwd_max_threads() {
  if (TPR == 0 && VPT == 2) return 768;
  if (TPR > 64) return 512;
  return (TPR != 0 && !BWD_COLS) ? 256 : 512;
}

// ------------------------------------------------------------------ forward, resident
// y = (x - mean) * inv_std * gamma + beta ; mean / inv_std saved per row.
// ROW_AFFINE: gamma / beta are indexed by (row % C) (channel-first InstanceNorm) instead
// of by column (LayerNorm).  y may alias x: a thread reads all of its vectors of a row
// before it writes any, and rows are never shared between lane groups.
//
// Statistics: the row is on chip, so the mean comes from one all-reduce of the sums and
// the variance from a second all-reduce of the squared deviations from that mean (the
// exact two-pass form, cheaper and more accurate than merging Welford triples across
// lanes); HBM sees the row once.
//
// RB rows per lane group form a batch; the next batch is loaded (software prefetch)
// before the current one is reduced, so loads overlap the arithmetic.
// EXACT: every lane owns exactly VPT vectors of every row of every batch (host-checked:
// D == lanes-per-row * VPT * V and n_rows % (rows-per-block * RB) == 0); all predicates
// fold away.
// RAGGED: D is not a multiple of V.  The lane after the last full vector takes the LAST V
// elements of the row (an access that overlaps its neighbour's, at element alignment) and
// uses only the D % V of them that no other lane owns; its stores are element-wise.
template <typename T, int V, int TPR, int VPT, int RB, bool EXACT, bool ROW_AFFINE,
          bool RAGGED = false>
__global__ void __launch_bounds__((resident_fwd_max_threads<TPR, VPT>()))
rows_fwd_resident(const T* x, const float* __restrict__ gamma, const float* __restrict__ beta,
                  T* y, float* __restrict__ mean_out, float* __restrict__ rstd_out,
                  int64_t n_rows, int d_elems, int C, float eps) {
  using M = RowMap<TPR>;
  constexpr int NE = V * VPT;
  static_assert(!(RAGGED && (EXACT || V == 1)), "ragged rows use the non-exact vector variants");
  // gamma / beta live in registers across rows unless that would exhaust the budget
  constexpr bool GB_REGS = !ROW_AFFINE && (VPT <= 8);
  static_assert(TPR != 0 || RB == 1, "row batching is for rows that fit one wave");
  __shared__ float red_buf[2][2][16];

  const int bdim = block_threads();
  const int n_waves = bdim / kWave;
  const int tpr = M::tpr(bdim);
  const int rpb = M::rows_per_block(bdim);
  const int lane_r = M::lane_in_row();
  const int slot = M::slot();
  const int64_t D = d_elems;
  const float inv_d = 1.0f / static_cast<float>(D);

  // Non-EXACT: loads are never predicated (a predicated load costs a full memory latency
  // of its own).  A vector slot beyond the row reads the row's last V elements, a row
  // beyond the batch reads the last row, and the values are masked out of the arithmetic.
  const int n_full = d_elems / V;
  const int rem = RAGGED ? d_elems % V : 0;
  bool vec_ok[VPT];
  int col[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = lane_r + k * tpr;
    const bool full = EXACT || idx < n_full;
    const bool tail = RAGGED && idx == n_full;
    vec_ok[k] = full || tail;
    col[k] = full ? idx * V : d_elems - V;
  }
  // RAGGED: the last vector of a row starts at D - V and repeats the elements 0 .. lo_t - 1 of
  // its neighbour.  It is vector k_tail of one lane of the row: the same k for every row (a
  // scalar), lo_t = 0 in every other lane.  All vectors are summed whole, by the code of an
  // unragged row, and under a uniform branch on k == k_tail the repeated elements are taken off
  // again (an error of the order of the rounding those elements cause in the sums anyway); y of
  // the repeated elements is computed and stored like every other: the same bits as the
  // neighbour's, from the same inputs.  Per-element ownership tests and guarded stores on every
  // vector cost the forward of [3355, 10004] 47 us instead of 32.
  const int k_tail = RAGGED ? n_full / tpr : -1;
  const int lo_t = (RAGGED && lane_r == n_full % tpr) ? V - rem : 0;
  auto elem_ok = [&](int r_ok, int k) -> bool {
    if constexpr (EXACT) return true;
    return vec_ok[k] && r_ok;
  };
  // A workgroup per row, row not a whole number of vectors per lane: a vector slot past the row
  // holds the row's last vector once more.  It is left out of the sums, a vector at a time, and
  // otherwise treated like every other, its store included (the same bits to the same address
  // as its owner's).  Stores under a condition would make the number of memory operations in
  // flight unknown to the compiler, whose waits for the current row then also wait for the
  // prefetched next one ([10000, 10232] halves 98.8 us against 76.0 us for [10000, 10240]).
  constexpr bool DUP_SLOTS = !EXACT && TPR == 0;

  float g[GB_REGS ? NE : 1], b[GB_REGS ? NE : 1];
  if constexpr (GB_REGS) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      float tg[V], tb[V];
      load_f32<V>(gamma + col[k], tg);
      load_f32<V>(beta + col[k], tb);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        g[k * V + i] = tg[i];
        b[k * V + i] = tb[i];
      }
    }
  }

  const int64_t stride = static_cast<int64_t>(gridDim.x) * rpb * RB;
  int64_t row0 = static_cast<int64_t>(blockIdx.x) * rpb * RB;

  // ROW_AFFINE: gamma / beta of a row's channel travel with the row's vectors (fetched at their
  // point of use, after the two reductions, they would cost a trip to L2 per row)
  struct RowAffine {
    float g[ROW_AFFINE ? RB : 1], b[ROW_AFFINE ? RB : 1];
  };
  auto load_batch = [&](int64_t base, Pack<T, V>(&raw)[RB][VPT], RowAffine& ra) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int64_t row_q = base + r * rpb + slot;
      const int64_t row = (EXACT || row_q < n_rows) ? row_q : n_rows - 1;
      const T* xr = x + row * D;
#pragma unroll
      for (int k = 0; k < VPT; ++k) raw[r][k] = load_pack<T, V>(xr + col[k]);
      if constexpr (ROW_AFFINE) {
        const int c = static_cast<int>(row % C);
        ra.g[r] = gamma[c];
        ra.b[r] = beta[c];
      }
    }
  };

  // prefetching doubles the raw-vector registers; long rows do without it
  constexpr bool PREFETCH = VPT * RB <= 4;
  auto process = [&](Pack<T, V>(&cur)[RB][VPT], const RowAffine& cur_ra, int64_t row0, int it) {
    bool row_ok[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) row_ok[r] = EXACT || row0 + r * rpb + slot < n_rows;
    // stage 1: convert once, sum; elements outside the row are kept at 0
    float f[RB][NE];
    float mean[RB], rstd[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        if constexpr (DUP_SLOTS) {
          float sv = 0.f;
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float v = to_f32(cur[r][k].v[i]);
            f[r][k * V + i] = v;
            sv += v;
          }
          if (RAGGED && k == k_tail) {
#pragma unroll
            for (int i = 0; i < V - 1; ++i) sv -= i < lo_t ? f[r][k * V + i] : 0.f;
          }
          s += vec_ok[k] ? sv : 0.f;
        } else {
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float v = elem_ok(row_ok[r], k) ? to_f32(cur[r][k].v[i]) : 0.f;
            f[r][k * V + i] = v;
            s += v;
          }
          if (RAGGED && k == k_tail) {
#pragma unroll
            for (int i = 0; i < V - 1; ++i) s -= i < lo_t ? f[r][k * V + i] : 0.f;
          }
        }
      }
      mean[r] = s;
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      if constexpr (TPR != 0) {
        mean[r] = group_sum<(TPR ? TPR : 1)>(mean[r]) * inv_d;
      } else {
        mean[r] = block_sum1(mean[r], red_buf[it & 1][0], n_waves) * inv_d;
      }
    }
    // stage 2: centre (exact second pass over registers), sum of squares
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      float q = 0.f;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        if constexpr (DUP_SLOTS) {
          float qv = 0.f;
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float d = f[r][k * V + i] - mean[r];
            f[r][k * V + i] = d;
            qv += d * d;
          }
          if (RAGGED && k == k_tail) {
#pragma unroll
            for (int i = 0; i < V - 1; ++i) qv -= i < lo_t ? f[r][k * V + i] * f[r][k * V + i] : 0.f;
          }
          q += vec_ok[k] ? qv : 0.f;
        } else {
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float d = elem_ok(row_ok[r], k) ? f[r][k * V + i] - mean[r] : 0.f;
            f[r][k * V + i] = d;
            q += d * d;
          }
          if (RAGGED && k == k_tail) {
#pragma unroll
            for (int i = 0; i < V - 1; ++i) q -= i < lo_t ? f[r][k * V + i] * f[r][k * V + i] : 0.f;
          }
        }
      }
      rstd[r] = q;
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      float q;
      if constexpr (TPR != 0) {
        q = group_sum<(TPR ? TPR : 1)>(rstd[r]);
      } else {
        q = block_sum1(rstd[r], red_buf[it & 1][1], n_waves);
      }
      rstd[r] = rsqrtf(q * inv_d + eps);
    }
    // stage 3: scale, shift, store
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int64_t row = row0 + r * rpb + slot;
      float gs = 1.f, bs = 0.f;
      if constexpr (ROW_AFFINE) {
        gs = cur_ra.g[r] * rstd[r];
        bs = cur_ra.b[r];
      }
      T* yr = y + row * D;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        float tg[V], tb[V];
        if constexpr (!ROW_AFFINE && !GB_REGS) {
          load_f32<V>(gamma + col[k], tg);
          load_f32<V>(beta + col[k], tb);
        }
        // (a workgroup per row never sees a row past the end)
        if (EXACT || DUP_SLOTS || (vec_ok[k] && row_ok[r])) {
          Pack<T, V> o;
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float d = f[r][k * V + i];
            float res;
            if constexpr (ROW_AFFINE) {
              res = d * gs + bs;
            } else if constexpr (GB_REGS) {
              res = d * (rstd[r] * g[k * V + i]) + b[k * V + i];
            } else {
              res = d * (rstd[r] * tg[i]) + tb[i];
            }
            o.v[i] = from_f32<T>(res);
          }
          store_pack<T, V>(yr + col[k], o);
        }
      }
      if (row_ok[r] && lane_r == 0) {
        mean_out[row] = mean[r];
        rstd_out[row] = rstd[r];
      }
    }
  };
  // Prefetch: the next batch is requested, under a condition, before the current one is worked
  // on.  (A loop that always requests and handles the last batch after it measured the same
  // once the first batch was made to arrive before the loop, see below, and is gone.)
  if constexpr (PREFETCH) {
    Pack<T, V> cur[RB][VPT];
    RowAffine cur_ra;
    if (row0 < n_rows) {
      load_batch(row0, cur, cur_ra);
      // The first batch is waited for here, outside the loop.  Otherwise the wait sits at the
      // batch's first use inside the loop, counted in memory operations still allowed in
      // flight as seen from this side of the loop's entry; on the way round the loop the
      // operations in flight there are the prefetch just issued, and that wait, needless then,
      // holds every row up for it ([10000, 10232] halves forward 98.8 us; 76.0 us for
      // [10000, 10240], whose instantiation happens to issue gamma / beta after the batch).
#pragma unroll
      for (int r = 0; r < RB; ++r) batch_loaded<T, V, VPT>(cur[r]);
      if constexpr (GB_REGS) {
        values_arrived(g);
        values_arrived(b);
      }
    }
    for (int it = 0; row0 < n_rows; row0 += stride, ++it) {
      Pack<T, V> nxt[RB][VPT];
      RowAffine nxt_ra;
      const bool more = row0 + stride < n_rows;
      if (more) load_batch(row0 + stride, nxt, nxt_ra);
      process(cur, cur_ra, row0, it);
      if (more) {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
#pragma unroll
          for (int k = 0; k < VPT; ++k) cur[r][k] = nxt[r][k];
        }
        cur_ra = nxt_ra;
      }
    }
  } else {
    for (int it = 0; row0 < n_rows; row0 += stride, ++it) {
      Pack<T, V> cur[RB][VPT];
      RowAffine cur_ra;
      load_batch(row0, cur, cur_ra);
      if constexpr (ROW_AFFINE) {
        // they are needed where the row's vectors are: not to be moved down to their use
#pragma unroll
        for (int r = 0; r < RB; ++r) asm volatile("" : "+v"(cur_ra.g[r]), "+v"(cur_ra.b[r]));
      }
      process(cur, cur_ra, row0, it);
    }
  }
}

// ----------------------------------------------------------------- backward, resident
// Per row, with xh = (x - mean) * r and g = dy * gamma:
//   s1 = sum g, s2 = sum g * xh, dx = r * (g - (s1 + xh * s2) / D)
// which is the reference's (2 (x - mean) dl_dvar + dl_dmu) / D + g r
// (fused_layer_norm_op.cu:84-88, norm_util.h:369-372,408-410) with
// dl_dvar = -1/2 r^3 sum g (x - mean), dl_dmu = -r s1.
//
// LayerNorm (ROW_AFFINE = false): every thread also accumulates, over all rows it
// visits, dgamma_j += dy * xh and dbeta_j += dy for the columns it owns; at the end the
// block folds them (lanes, then waves through LDS, fixed order) and writes ONE partial
// row part[blockIdx.x][0][0..D) (dgamma) and part[blockIdx.x][1][0..D) (dbeta); a second
// kernel sums the partial rows.  `part` has gridDim.x * 2 * D floats.
//
// InstanceNorm channel-first (ROW_AFFINE = true): gamma is the scalar of channel
// row % C, the two row sums a = sum dy, b = sum dy * xh give s1 = gamma a, s2 = gamma b and
// are written to part[n][0][c] = b, part[n][1][c] = a  (n = row / C), i.e. `part` has
// N * 2 * C floats and the same second kernel folds it over n.
// dx may alias dy (a thread reads its elements of a row before it writes them), not x.
// RB / EXACT / prefetch as in the forward kernel.
// Channel-first InstanceNorm with a workgroup per plane: the fold of the per-plane sums over the
// batch (dgamma[c] = sum over n of the plane sums of (n, c)) can run inside the row kernel instead
// of as a launch of its own.  Every workgroup publishes the two sums of its plane as a tagged
// pair as soon as it has them, before it computes and stores dx; after its own planes, one of the
// last workgroups of the grid waits (a lane per instance, a bounded number of polls) for the N
// pairs of channel c and adds them up.  The host asks for it only when the planes of a channel are
// all handled on one XCD, the folding workgroup's (a workgroup per plane: C and the grid multiples
// of the XCD count, plane n * C + c goes to workgroup (n * C + c) mod grid; q planes per workgroup
// and step: C / q and the grid multiples of it), so that plain stores are visible to the
// device-scope polls, when N <= 64, dx != dy and the stream is not being captured.  A workgroup
// whose wait runs out recomputes the sums of the N planes itself, with the code the row loop uses
// (same bits).
constexpr int kAffineFoldMaxStep = 64;     // planes per workgroup and step (lane groups per plane)
constexpr int kAffineFoldMaxPairs = 1024;  // instances x planes per step that the fallback keeps in LDS
struct AffineFold {
  cl_word* tagged = nullptr;  // [N * C] pairs (sum dy * xh, sum dy); nullptr: col_reduce follows
  float* dgamma = nullptr;
  float* dbeta = nullptr;
  unsigned tag = 0;
  int max_polls = 0;
  int N = 0;
};

template <typename T, int V, int TPR, int VPT, int RB, bool EXACT, bool ROW_AFFINE,
          bool RAGGED = false>
__global__ void __launch_bounds__((resident_bwd_max_threads<TPR, !ROW_AFFINE, RB, VPT>()))
rows_bwd_resident(const T* dy, const T* __restrict__ x,
                  const float* __restrict__ gamma, const float* __restrict__ mean_in,
                  const float* __restrict__ rstd_in, T* dx,
                  float* __restrict__ part, int64_t n_rows, int d_elems, int C, AffineFold fold) {
  using M = RowMap<TPR>;
  constexpr int NE = V * VPT;
  static_assert(!(RAGGED && (EXACT || V == 1)), "ragged rows use the non-exact vector variants");
  static_assert((TPR != 0 && TPR <= kWave) || RB == 1, "row batching is for rows that fit one wave");
  __shared__ float2 sum_buf[2][16];
  // LayerNorm only: waves x fold_groups_per_pass x min(TPR, 64) x W floats
  extern __shared__ __attribute__((aligned(16))) float fold_buf[];

  const int bdim = block_threads();
  const int n_waves = bdim / kWave;
  const int tpr = M::tpr(bdim);
  const int rpb = M::rows_per_block(bdim);
  const int lane_r = M::lane_in_row();
  const int slot = M::slot();
  const int64_t D = d_elems;
  const float inv_d = 1.0f / static_cast<float>(D);

  // Non-EXACT / RAGGED: unpredicated loads from clamped positions, masked arithmetic (see
  // the forward kernel).
  const int n_full = d_elems / V;
  const int rem = RAGGED ? d_elems % V : 0;
  bool vec_ok[VPT];
  int col[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = lane_r + k * tpr;
    const bool full = EXACT || idx < n_full;
    const bool tail = RAGGED && idx == n_full;
    vec_ok[k] = full || tail;
    col[k] = full ? idx * V : d_elems - V;
  }
  // RAGGED: as in the forward kernel, the overlapping last vector (vector k_tail, a scalar, of
  // one lane; lo_t repeated elements there, 0 elsewhere) is summed whole and its repeated
  // elements are taken off the row sums under a uniform branch; dx of the repeated elements is
  // computed and stored like every other (the neighbour's bits); their dgamma / dbeta
  // accumulators are simply not written out.
  const int k_tail = RAGGED ? n_full / tpr : -1;
  const int lo_t = (RAGGED && lane_r == n_full % tpr) ? V - rem : 0;

  float g[ROW_AFFINE ? 1 : NE];
  float acc_g[ROW_AFFINE ? 1 : NE], acc_b[ROW_AFFINE ? 1 : NE];
  if constexpr (!ROW_AFFINE) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      float tg[V];
      load_f32<V>(gamma + col[k], tg);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        g[k * V + i] = tg[i];
        acc_g[k * V + i] = 0.f;
        acc_b[k * V + i] = 0.f;
      }
    }
  }

  const int64_t stride = static_cast<int64_t>(gridDim.x) * rpb * RB;
  int64_t row0 = static_cast<int64_t>(blockIdx.x) * rpb * RB;

  struct Batch {
    Pack<T, V> px[RB][VPT], pd[RB][VPT];
    float mean[RB], rstd[RB];
    float gm[ROW_AFFINE ? RB : 1];  // ROW_AFFINE: gamma of the row's channel, fetched with the row
  };
  auto load_batch = [&](int64_t base, Batch& t) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int64_t row_q = base + r * rpb + slot;
      const int64_t row = (EXACT || row_q < n_rows) ? row_q : n_rows - 1;
      const T* xr = x + row * D;
      const T* dyr = dy + row * D;
      t.mean[r] = mean_in[row];
      t.rstd[r] = rstd_in[row];
      if constexpr (ROW_AFFINE) t.gm[r] = gamma[static_cast<int>(row % C)];
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        t.px[r][k] = load_pack_last<T, V>(xr + col[k]);
        t.pd[r][k] = load_pack_last<T, V>(dyr + col[k]);
      }
    }
  };

  // (a channel-first plane per workgroup: the launch has a workgroup per plane or nearly, no next
  // row to request, and the extra registers cost a wave per SIMD)
  constexpr bool PREFETCH = VPT * RB <= (TPR == 0 && ROW_AFFINE ? 2 : 4);
  // A workgroup per row whose row is not a whole number of vectors per lane: as in the forward
  // kernel, a vector slot past the row holds the row's last vector again, and is masked out of
  // the row sums only; dx of it is stored like every other (the same bits as its owner's).
  constexpr bool DUP_SLOTS = !EXACT && TPR == 0;
  // stage 1: convert once; xh = (x - mean) * r, gv = dy * gamma; row sums and the
  // column accumulators.  Elements outside the row are 0 and add nothing.
  auto row_sums = [&](Batch& cur, const bool (&row_ok)[RB], float (&xh)[RB][NE], float (&gv)[RB][NE],
                      float (&s1)[RB], float (&s2)[RB], int it) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      float a1 = 0.f, a2 = 0.f;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        // DUP_SLOTS: the vector is worked on whatever it is and only its share of the row
        // sums is dropped (its column accumulators are never written out)
        float v1 = 0.f, v2 = 0.f;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const int e = k * V + i;
          const bool ok = EXACT || DUP_SLOTS || (vec_ok[k] && row_ok[r]);
          const float h = ok ? (to_f32(cur.px[r][k].v[i]) - cur.mean[r]) * cur.rstd[r] : 0.f;
          const float d = ok ? to_f32(cur.pd[r][k].v[i]) : 0.f;
          xh[r][e] = h;
          if constexpr (ROW_AFFINE) {
            gv[r][e] = d;
            v1 += d;
            v2 += d * h;
          } else {
            const float t = d * g[e];
            gv[r][e] = t;
            v1 += t;
            v2 += t * h;
            acc_g[e] += d * h;
            acc_b[e] += d;
          }
        }
        if (RAGGED && k == k_tail) {
#pragma unroll
          for (int i = 0; i < V - 1; ++i) {
            v1 -= i < lo_t ? gv[r][k * V + i] : 0.f;
            v2 -= i < lo_t ? gv[r][k * V + i] * xh[r][k * V + i] : 0.f;
          }
        }
        a1 += DUP_SLOTS && !vec_ok[k] ? 0.f : v1;
        a2 += DUP_SLOTS && !vec_ok[k] ? 0.f : v2;
      }
      s1[r] = a1;
      s2[r] = a2;
    }
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      if constexpr (TPR > kWave) {
        const float2 t = wavegroup_sum2<TPR / kWave>(s1[r], s2[r], sum_buf[it & 1]);
        s1[r] = t.x;
        s2[r] = t.y;
      } else if constexpr (TPR != 0) {
        s1[r] = group_sum<(TPR && TPR <= kWave ? TPR : 1)>(s1[r]);
        s2[r] = group_sum<(TPR && TPR <= kWave ? TPR : 1)>(s2[r]);
      } else {
        const float2 t = block_sum2(s1[r], s2[r], sum_buf[it & 1], n_waves);
        s1[r] = t.x;
        s2[r] = t.y;
      }
    }
  };
  auto process = [&](Batch& cur, int64_t row0, int it) {
    bool row_ok[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) row_ok[r] = EXACT || row0 + r * rpb + slot < n_rows;
    float xh[RB][NE], gv[RB][NE];
    float s1[RB], s2[RB];
    row_sums(cur, row_ok, xh, gv, s1, s2, it);
    // stage 2: dx = scale * gv + (A * xh + B), A = -scale * s2 / D, B = -scale * s1 / D
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      const int64_t row = row0 + r * rpb + slot;
      float scale = cur.rstd[r];
      if constexpr (ROW_AFFINE) {
        scale *= cur.gm[r];
        if (row_ok[r] && lane_r == 0) {
          if (fold.tagged != nullptr) {
            cl_publish(fold.tagged + row * 2, s2[r], s1[r], fold.tag);
          } else {
            const int64_t n = row / C;
            const int c = static_cast<int>(row % C);
            part[(n * 2 + 0) * C + c] = s2[r];
            part[(n * 2 + 1) * C + c] = s1[r];
          }
        }
      }
      const float ca = -scale * (s2[r] * inv_d), cb = -scale * (s1[r] * inv_d);
      T* dxr = dx + row * D;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        if (EXACT || DUP_SLOTS || (vec_ok[k] && row_ok[r])) {
          Pack<T, V> o;
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const int e = k * V + i;
            o.v[i] = from_f32<T>(scale * gv[r][e] + (ca * xh[r][e] + cb));
          }
          store_pack<T, V>(dxr + col[k], o);
        }
      }
    }
  };
  // the first batch and gamma are waited for before the loop (see values_arrived)
  auto first_batch_arrived = [&](Batch& t) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
      batch_loaded<T, V, VPT>(t.px[r]);
      batch_loaded<T, V, VPT>(t.pd[r]);
    }
    values_arrived(t.mean);
    values_arrived(t.rstd);
    if constexpr (ROW_AFFINE) {
      values_arrived(t.gm);
    } else {
      values_arrived(g);
    }
  };
  if constexpr (PREFETCH) {
    Batch cur;
    if (row0 < n_rows) {
      load_batch(row0, cur);
      first_batch_arrived(cur);
    }
    for (int it = 0; row0 < n_rows; row0 += stride, ++it) {
      Batch nxt;
      const bool more = row0 + stride < n_rows;
      if (more) load_batch(row0 + stride, nxt);
      process(cur, row0, it);
      if (more) cur = nxt;
    }
  } else {
    for (int it = 0; row0 < n_rows; row0 += stride, ++it) {
      Batch cur;
      load_batch(row0, cur);
      if constexpr (ROW_AFFINE) {
        // needed where the row's vectors are: not to be moved down to its use
#pragma unroll
        for (int r = 0; r < RB; ++r) asm volatile("" : "+v"(cur.gm[r]));
      }
      process(cur, row0, it);
    }
  }

  if constexpr (ROW_AFFINE && TPR == 0) {
    if (fold.tagged != nullptr) {
      // dgamma / dbeta of channel c are folded by workgroup G-1 - (C-1-c) % G: the workgroups
      // that start last, so that every plane they wait for belongs to a workgroup that has been
      // started already (a grid larger than the chip holds at once would otherwise leave its
      // first workgroups waiting in the places that their peers need), and one whose index is
      // congruent to c modulo the XCD count (C and G are multiples of it), as the indices of
      // the workgroups that publish the planes of channel c are.
      __shared__ int fold_failed;
      __shared__ float inst[kWave][2];
      const int lane = threadIdx.x & (kWave - 1);
      const int wave = threadIdx.x / kWave;
      const int N = fold.N;
      int it = 0;
      for (int64_t c = static_cast<int64_t>(C) - static_cast<int64_t>(gridDim.x) + blockIdx.x; c >= 0; c -= gridDim.x) {
        if (wave == 0) {
          float pb, pa;
          const bool ok = cl_wait_pair(fold.tagged + (static_cast<int64_t>(lane < N ? lane : 0) * C + c) * 2,
                                       lane < N, fold.tag, fold.max_polls, pb, pa);
          if (ok) {
            const float b = group_sum<kWave>(lane < N ? pb : 0.f);
            const float a = group_sum<kWave>(lane < N ? pa : 0.f);
            if (lane == 0) {
              fold.dgamma[c] = b;
              fold.dbeta[c] = a;
            }
          }
          if (lane == 0) fold_failed = ok ? 0 : 1;
        }
        __syncthreads();
        if (fold_failed) {  // uniform: the planes of channel c, summed here as their workgroups sum them
          for (int n = 0; n < N; ++n) {
            Batch t;
            load_batch(static_cast<int64_t>(n) * C + c, t);
            bool row_ok[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r) row_ok[r] = true;
            float xh[RB][NE], gv[RB][NE];
            float s1[RB], s2[RB];
            row_sums(t, row_ok, xh, gv, s1, s2, it++);
            if (threadIdx.x == 0) {
              inst[n][0] = s2[0];
              inst[n][1] = s1[0];
            }
          }
          __syncthreads();
          if (wave == 0) {
            const float b = group_sum<kWave>(lane < N ? inst[lane < N ? lane : 0][0] : 0.f);
            const float a = group_sum<kWave>(lane < N ? inst[lane < N ? lane : 0][1] : 0.f);
            if (lane == 0) {
              fold.dgamma[c] = b;
              fold.dbeta[c] = a;
            }
          }
        }
        __syncthreads();
      }
    }
  }
  if constexpr (ROW_AFFINE && TPR != 0) {
    if (fold.tagged != nullptr) {
      // Lane groups per plane: a workgroup takes q = rpb * RB consecutive planes per step, i.e.
      // the channels j * q .. j * q + q - 1 of an instance (C is a multiple of q), and so does the
      // fold: channel group j belongs to workgroup G-1 - (C/q-1-j) % G, which is started after
      // every workgroup that handles planes of the group and sits on their XCD (C / q and G
      // multiples of the XCD count and one of the other).  A wave per channel, a lane per instance.
      __shared__ int fold_fail[kAffineFoldMaxStep];
      __shared__ float inst[kAffineFoldMaxPairs][2];
      const int lane = threadIdx.x & (kWave - 1);
      const int wave = threadIdx.x / kWave;
      const int N = fold.N;
      const int q = rpb * RB;
      const int64_t groups = C / q;
      int it = 0;
      for (int64_t j = groups - static_cast<int64_t>(gridDim.x) + blockIdx.x; j >= 0; j -= gridDim.x) {
        const int c0 = static_cast<int>(j) * q;
        if (static_cast<int>(threadIdx.x) < q) fold_fail[threadIdx.x] = 0;
        __syncthreads();
        for (int i = wave; i < q; i += n_waves) {
          float pb, pa;
          const bool ok = cl_wait_pair(fold.tagged + (static_cast<int64_t>(lane < N ? lane : 0) * C + c0 + i) * 2,
                                       lane < N, fold.tag, fold.max_polls, pb, pa);
          if (ok) {
            const float b = group_sum<kWave>(lane < N ? pb : 0.f);
            const float a = group_sum<kWave>(lane < N ? pa : 0.f);
            if (lane == 0) {
              fold.dgamma[c0 + i] = b;
              fold.dbeta[c0 + i] = a;
            }
          } else if (lane == 0) {
            fold_fail[i] = 1;
          }
        }
        __syncthreads();
        bool failed = false;
        for (int i = 0; i < q; ++i) failed = failed || fold_fail[i] != 0;
        if (failed) {  // uniform: the planes of these channels, summed here as their workgroups sum them
          for (int n = 0; n < N; ++n) {
            Batch t;
            load_batch(static_cast<int64_t>(n) * C + c0, t);
            bool row_ok[RB];
#pragma unroll
            for (int r = 0; r < RB; ++r) row_ok[r] = true;
            float xh[RB][NE], gv[RB][NE];
            float s1[RB], s2[RB];
            row_sums(t, row_ok, xh, gv, s1, s2, it++);
            if (lane_r == 0) {
#pragma unroll
              for (int r = 0; r < RB; ++r) {
                inst[n * q + r * rpb + slot][0] = s2[r];
                inst[n * q + r * rpb + slot][1] = s1[r];
              }
            }
          }
          __syncthreads();
          for (int i = wave; i < q; i += n_waves) {
            if (fold_fail[i]) {
              const float b = group_sum<kWave>(lane < N ? inst[(lane < N ? lane : 0) * q + i][0] : 0.f);
              const float a = group_sum<kWave>(lane < N ? inst[(lane < N ? lane : 0) * q + i][1] : 0.f);
              if (lane == 0) {
                fold.dgamma[c0 + i] = b;
                fold.dbeta[c0 + i] = a;
              }
            }
          }
        }
        __syncthreads();
      }
    }
  }
  if constexpr (!ROW_AFFINE) {
    float* prow = part + static_cast<int64_t>(blockIdx.x) * 2 * D;
    if constexpr (TPR == 0) {
      // one row per block: every thread owns its columns outright
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        if (vec_ok[k]) {
          float tg[V], tb[V];
#pragma unroll
          for (int i = 0; i < V; ++i) {
            tg[i] = acc_g[k * V + i];
            tb[i] = acc_b[k * V + i];
          }
          if (RAGGED && k == k_tail) {
            store_f32_from<V>(prow + col[k], tg, lo_t);
            store_f32_from<V>(prow + D + col[k], tb, lo_t);
          } else {
            store_f32<V>(prow + col[k], tg);
            store_f32<V>(prow + D + col[k], tb);
          }
        }
      }
    } else {
      // 1) fold the row slots that share a wave (lanes l, l+TPR, ... own the same columns)
      if constexpr (TPR < kWave && TPR != 0) {
#pragma unroll
        for (int i = 0; i < NE; ++i) {
#pragma unroll
          for (int m = (TPR ? TPR : 1); m < kWave; m <<= 1) {
            acc_g[i] += lane_xor(acc_g[i], m);
            acc_b[i] += lane_xor(acc_b[i], m);
          }
        }
      }
      // 2) fold the waves through LDS: every wave leaves its sums there, ONE barrier, and every
      //    thread of the workgroup then adds one output (W adjacent columns of dgamma or of
      //    dbeta) over the waves that hold it, in wave order, and stores it to the partial row.
      //    (A pairwise tree, upper half of the waves writing and lower half adding, moves a little
      //    less data but takes six barriers for eight waves, leaves most waves idle and the
      //    whole store to one wave: measured 1.2 us of a 12.2 us kernel at [8192, 1024].)
      //    The sums of a lane travel as Q groups of W floats (W = 4: 16-byte LDS accesses); at
      //    most QC groups per pass keep the buffer within 64 KiB for eight waves.
      constexpr int WPG = TPR > kWave ? TPR / kWave : 1;  // waves per row
      constexpr int LR = TPR < kWave ? TPR : kWave;       // lanes of a wave that hold sums
      constexpr int W = fold_width<V>();
      constexpr int Q = 2 * NE / W;
      constexpr int QC = fold_groups_per_pass<V, VPT, TPR>();
      const int lane = threadIdx.x & (kWave - 1);
      const int wave = threadIdx.x / kWave;
      float vals[2 * NE];
#pragma unroll
      for (int i = 0; i < NE; ++i) {
        vals[i] = acc_g[i];
        vals[NE + i] = acc_b[i];
      }
#pragma unroll
      for (int c0 = 0; c0 < Q; c0 += QC) {
        const int qn = Q - c0 < QC ? Q - c0 : QC;
        if (c0 > 0) __syncthreads();  // the previous pass has been read
        if (LR == kWave || lane < LR) {
#pragma unroll
          for (int q = 0; q < QC; ++q) {
            if (q < qn) {
              float* dst = fold_buf + (static_cast<size_t>(wave * qn + q) * LR + lane) * W;
#pragma unroll
              for (int j = 0; j < W; ++j) dst[j] = vals[(c0 + q) * W + j];
            }
          }
        }
        __syncthreads();
        const int n_out = WPG * qn * LR;
        for (int o = static_cast<int>(threadIdx.x); o < n_out; o += bdim) {
          const int ol = o % LR;
          const int oq = (o / LR) % qn;
          const int og = o / (LR * qn);  // part of the row (wave of its wave group)
          float sum[W];
          {
            const float* src = fold_buf + (static_cast<size_t>(og * qn + oq) * LR + ol) * W;
#pragma unroll
            for (int j = 0; j < W; ++j) sum[j] = src[j];
          }
          for (int w = og + WPG; w < n_waves; w += WPG) {
            const float* src = fold_buf + (static_cast<size_t>(w * qn + oq) * LR + ol) * W;
#pragma unroll
            for (int j = 0; j < W; ++j) sum[j] += src[j];
          }
          // where the W sums go: element e0 of the lane's 2 * NE sums
          const int e0 = (c0 + oq) * W;
          const int which = e0 >= NE ? 1 : 0;  // 0: dgamma terms, 1: dbeta terms
          const int e = e0 - which * NE;
          const int k = e / V, i0 = e % V;
          const int idx = og * kWave + ol + k * tpr;  // vector of the row
          const bool full = EXACT || idx < n_full;
          const bool tail = RAGGED && idx == n_full;
          if (full || tail) {
            const int ocol = full ? idx * V : d_elems - V;
            const int olo = tail ? V - rem : 0;
            float* dst = prow + static_cast<int64_t>(which) * D + ocol + i0;
            if (!RAGGED || olo == 0) {
              store_f32<W>(dst, sum);
            } else {
#pragma unroll
              for (int j = 0; j < W; ++j) {
                if (i0 + j >= olo) dst[j] = sum[j];
              }
            }
          }
        }
      }
    }
  }
}

// ------------------------------------------- backward, resident, accumulators in LDS
// LayerNorm rows too long for rows_bwd_resident, whose per-lane dgamma / dbeta accumulators
// cost two registers per element held: the same single pass (a workgroup per row, x and dy
// read once, one partial row per workgroup for col_reduce), with the accumulators of the
// workgroup's columns in LDS instead, acc[0][0..D) (dgamma terms) and acc[1][0..D) (dbeta
// terms): 8 * D bytes, so D <= 20416 on the 160 KiB of a gfx950 CU (one workgroup per CU).
// A thread owns its columns outright (one row per workgroup), so nobody else touches its
// LDS words and the accumulation needs no barrier; per row it reads and writes 16 * D
// bytes of LDS per workgroup, about a sixth of the time the CU's share of the memory
// bandwidth needs for the row.  xh and g are recomputed from the raw vectors for the dx
// pass instead of being kept.  4 vectors per lane on up to 640 (16-bit) / 1024 (float32) threads;
// with 8 per lane on at most 512 threads a CU has too few waves ([8192, 18432] fp16 226 -> 202 us).
// dx may alias dy, not x.
constexpr int kBwdLdsThreads = 512;
constexpr int kBwdLdsVpt = 8;
// Largest workgroup of a rows_bwd_lds<.., VPT> launch: rows of at most 20416 elements (the LDS
// limit) and 4096 vectors.  16-bit rows at 4 vectors per lane: 2552 vectors on 640 threads.
template <int V, int VPT>
constexpr int bwd_lds_max_threads() {
  return VPT == 8 ? kBwdLdsThreads : (V == 8 ? 640 : 1024);
}

template <typename T, int V, bool RAGGED, int VPT = kBwdLdsVpt>
__global__ void __launch_bounds__((bwd_lds_max_threads<V, VPT>()))
rows_bwd_lds(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
             const float* __restrict__ mean_in, const float* __restrict__ rstd_in, T* dx,
             float* __restrict__ part, int64_t n_rows, int d_elems) {
  __shared__ float2 sum_buf[2][16];
  extern __shared__ __attribute__((aligned(16))) float acc[];  // [2][d_elems rounded up to 4]
  float* const acc_b = acc + (d_elems + 3) / 4 * 4;
  const int bdim = block_threads();
  const int n_waves = bdim / kWave;
  const int64_t D = d_elems;
  const float inv_d = 1.0f / static_cast<float>(D);
  const int n_full = d_elems / V;
  const int rem = RAGGED ? d_elems % V : 0;
  // unpredicated loads from clamped positions, masked arithmetic (as in rows_bwd_resident)
  bool vec_ok[VPT];
  int col[VPT];
  int lds_col[VPT];  // where a FULL vector's accumulators sit: a multiple of V, which lets the
                     // compiler use 16-byte LDS accesses (col[k] may be D - V)
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int idx = static_cast<int>(threadIdx.x) + k * bdim;
    const bool full = idx < n_full;
    const bool tail = RAGGED && idx == n_full;
    vec_ok[k] = full || tail;
    col[k] = full ? idx * V : d_elems - V;
    lds_col[k] = idx * V;
  }
  // RAGGED: the overlapping last vector is vector k_tail (a scalar) of one thread, which owns
  // only its elements lo_t .. V-1 (lo_t = 0 in every other thread).  Vector k_tail takes its sums
  // and adds to the LDS accumulators element by element (the repeated elements' accumulators are
  // the neighbour's), under a uniform branch; every other vector runs the code of an unragged
  // row, and dx of the repeated elements is stored like every other (the neighbour's bits).
  const int k_tail = RAGGED ? n_full / bdim : -1;
  const int lo_t = (RAGGED && static_cast<int>(threadIdx.x) == n_full % bdim) ? V - rem : 0;
  float g[VPT][V];
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    load_f32<V>(gamma + col[k], g[k]);
    if (vec_ok[k]) {
      if (RAGGED && k == k_tail && lo_t != 0) {
#pragma unroll
        for (int i = 0; i < V; ++i) {
          if (i >= lo_t) {
            acc[col[k] + i] = 0.f;
            acc_b[col[k] + i] = 0.f;
          }
        }
      } else {
        const float zero[V] = {};
        store_f32<V>(acc + lds_col[k], zero);
        store_f32<V>(acc_b + lds_col[k], zero);
      }
    }
  }
  // PREFETCH (4 vectors per lane): the next row's vectors are requested before the current row
  // is worked on; the first row and gamma arrive before the loop (see values_arrived).  The
  // 16-bit instantiations then sit at their register limit (168 of 170 for 640 threads) and
  // spill 5 to 10 values; [8192, 18432] halves still 191 -> 178 us, [2048, 18432] 65 -> 59 us
  // (requesting the row later, behind the accumulation, spills the same).  float32: no spill,
  // and no difference either.
  constexpr bool PREFETCH = VPT <= 4;
  auto load_row = [&](int64_t row, Pack<T, V>(&qx)[VPT], Pack<T, V>(&qd)[VPT]) {
    const T* xr = x + row * D;
    const T* dyr = dy + row * D;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      qx[k] = load_pack_last<T, V>(xr + col[k]);
      qd[k] = load_pack_last<T, V>(dyr + col[k]);
    }
  };
  Pack<T, V> px[VPT], pd[VPT];
  if constexpr (PREFETCH) {
    if (static_cast<int64_t>(blockIdx.x) < n_rows) {
      load_row(blockIdx.x, px, pd);
      batch_loaded<T, V, VPT>(px);
      batch_loaded<T, V, VPT>(pd);
#pragma unroll
      for (int k = 0; k < VPT; ++k) values_arrived(g[k]);
    }
  }
  int it = 0;
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x, ++it) {
    const float mean = mean_in[row], rstd = rstd_in[row];
    Pack<T, V> nx[PREFETCH ? VPT : 1], nd[PREFETCH ? VPT : 1];
    const bool more = PREFETCH && row + gridDim.x < n_rows;
    if constexpr (PREFETCH) {
      if (more) load_row(row + gridDim.x, nx, nd);
    } else {
      load_row(row, px, pd);
      batch_loaded<T, V, VPT>(px);
      batch_loaded<T, V, VPT>(pd);
    }
    float a1 = 0.f, a2 = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      if (vec_ok[k]) {
        if (RAGGED && k == k_tail && lo_t != 0) {  // the one thread that holds the last vector
#pragma unroll
          for (int i = 0; i < V; ++i) {
            if (i >= lo_t) {
              const float h = (to_f32(px[k].v[i]) - mean) * rstd;
              const float d = to_f32(pd[k].v[i]);
              const float t = d * g[k][i];
              a1 += t;
              a2 += t * h;
              acc[col[k] + i] += d * h;
              acc_b[col[k] + i] += d;
            }
          }
        } else {
          float tg[V], tb[V];
          load_f32<V>(acc + lds_col[k], tg);
          load_f32<V>(acc_b + lds_col[k], tb);
#pragma unroll
          for (int i = 0; i < V; ++i) {
            const float h = (to_f32(px[k].v[i]) - mean) * rstd;
            const float d = to_f32(pd[k].v[i]);
            const float t = d * g[k][i];
            a1 += t;
            a2 += t * h;
            tg[i] += d * h;
            tb[i] += d;
          }
          store_f32<V>(acc + lds_col[k], tg);
          store_f32<V>(acc_b + lds_col[k], tb);
        }
      }
      // one vector's accumulators at a time: with the LDS reads of all eight vectors moved to
      // the front, the kernel does not fit its registers
      asm volatile("" ::: "memory");
    }
    // (only the raw vectors wait through the reduction; xh and g are computed again)
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      forget_derived(px[k]);
      forget_derived(pd[k]);
    }
    const float2 s = block_sum2(a1, a2, sum_buf[it & 1], n_waves);
    const float ca = -rstd * (s.y * inv_d), cb = -rstd * (s.x * inv_d);
    T* dxr = dx + row * D;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      if (vec_ok[k]) {
        Pack<T, V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float h = (to_f32(px[k].v[i]) - mean) * rstd;
          const float t = to_f32(pd[k].v[i]) * g[k][i];
          o.v[i] = from_f32<T>(rstd * t + (ca * h + cb));
        }
        store_pack<T, V>(dxr + col[k], o);
      }
    }
    if constexpr (PREFETCH) {
      if (more) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
          px[k] = nx[k];
          pd[k] = nd[k];
        }
      }
    }
  }
  // the workgroup's partial row: every thread copies the columns it owns
  float* prow = part + static_cast<int64_t>(blockIdx.x) * 2 * D;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    if (vec_ok[k]) {
      if (RAGGED && k == k_tail && lo_t != 0) {
#pragma unroll
        for (int i = 0; i < V; ++i) {
          if (i >= lo_t) {
            prow[col[k] + i] = acc[col[k] + i];
            prow[D + col[k] + i] = acc_b[col[k] + i];
          }
        }
      } else {
        float tg[V], tb[V];
        load_f32<V>(acc + lds_col[k], tg);
        load_f32<V>(acc_b + lds_col[k], tb);
        store_f32<V>(prow + lds_col[k], tg);
        store_f32<V>(prow + D + lds_col[k], tb);
      }
    }
  }
}

// ------------------------------------- rows staged in registers and LDS, single pass
// Rows longer than the register-resident kernels take (4096 vectors) but short enough to sit on
// chip in one workgroup: the first kStagedRegVec vectors of every thread stay in registers,
// the rest of the row waits in LDS as raw 16-byte vectors (up to 152 KiB of a gfx950 CU's
// 160), and the row still makes ONE trip through memory: exact two-pass statistics and the
// normalisation read the staged copy.  A thread only ever reads back the LDS words it wrote
// itself, so the staging needs no barrier; the two block-wide sums are the only ones.
// Channel-first InstanceNorm planes (gamma / beta are scalars of the row; LayerNorm's per-column
// gamma / beta would be read again for every row, three times the bytes of the row itself from
// L2: measured slower than the 2-D tiles): forward up to 27 vectors per thread (110592 halves:
// a 48^3 or 256^2 plane), backward (x and dy staged) up to 17 (69632 halves).  The two-stage
// kernels (split_*) read such planes twice.
constexpr int kStagedThreads = 512;
constexpr int kStagedRegVec = 8;

// Where vector slot idx of a row lies: its first column (clamped to a valid one when the slot
// is past the row) and whether it holds data.  The last vector of a ragged row starts at D - V,
// so its first V - D % V elements repeat the last elements of its neighbour: the sums take it
// whole and the repeated elements are taken off again, once per row, by the thread that holds
// it (it always sits in the LDS part: slot D / V >= 4096); the outputs of the repeated elements
// are stored like every other, the same bits as the neighbour's from the same inputs.
template <int V>
struct StagedSlot {
  int col;
  bool ok;
};
template <int V>
__device__ __forceinline__ StagedSlot<V> staged_slot(int idx, int d_elems) {
  const int n_full = d_elems / V;
  const int rem = d_elems % V;
  StagedSlot<V> s;
  const bool full = idx < n_full;
  const bool tail = rem != 0 && idx == n_full;
  s.ok = full || tail;
  s.col = full ? idx * V : (tail ? d_elems - V : 0);
  return s;
}

// The staged copy is kept as 16-byte register quads (one LDS access each).
template <typename T, int V>
__device__ __forceinline__ u32x4 pack_bits(const Pack<T, V>& v) {
  static_assert(sizeof(T) * V == 16, "staged rows are rows of 16-byte vectors");
  u32x4 b;
  __builtin_memcpy(&b, &v, 16);
  return b;
}
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> bits_pack(const u32x4& b) {
  Pack<T, V> v;
  __builtin_memcpy(&v, &b, 16);
  return v;
}

template <typename T, int V>
__global__ void __launch_bounds__(kStagedThreads)
rows_fwd_staged(const T* x, const float* __restrict__ gamma, const float* __restrict__ beta, T* y,
                float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t n_rows,
                int d_elems, int C, float eps, int nv_lds) {
  constexpr int R = kStagedRegVec;
  constexpr int B = 8;  // vectors per thread whose loads are in flight together (16 measured slower)
  constexpr int NW = kStagedThreads / kWave;
  __shared__ float red[2][16];
  extern __shared__ __attribute__((aligned(16))) unsigned char staged_bytes[];
  u32x4* stage = reinterpret_cast<u32x4*>(staged_bytes);  // [nv_lds][kStagedThreads]
  const int tid = static_cast<int>(threadIdx.x);
  const int64_t D = d_elems;
  const float inv_d = 1.0f / static_cast<float>(D);
  StagedSlot<V> rs[R];
#pragma unroll
  for (int j = 0; j < R; ++j) rs[j] = staged_slot<V>(tid + j * kStagedThreads, d_elems);
  auto lds_slot = [&](int j) { return staged_slot<V>(tid + (R + j) * kStagedThreads, d_elems); };
  // ragged rows: the LDS slot of the overlapping last vector and, in the thread that holds it,
  // the number of elements it repeats
  const bool ragged = d_elems % V != 0;
  const int j_tail = ragged ? (d_elems / V) / kStagedThreads - R : 0;
  const int lo_t = (ragged && tid == (d_elems / V) % kStagedThreads) ? V - d_elems % V : 0;

  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    const T* xr = x + row * D;
    T* yr = y + row * D;
    // ---- load: registers first, then the LDS part in batches; the sum on the way
    Pack<T, V> reg[R];
#pragma unroll
    for (int j = 0; j < R; ++j) reg[j] = load_pack<T, V>(xr + rs[j].col);
    float sum = 0.f;
    for (int j0 = 0; j0 < nv_lds; j0 += B) {
      Pack<T, V> pk[B];
      StagedSlot<V> sl[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        sl[u] = lds_slot(j0 + u < nv_lds ? j0 + u : nv_lds - 1);
        pk[u] = load_pack<T, V>(xr + sl[u].col);
      }
      batch_loaded<T, V, B>(pk);
#pragma unroll
      for (int u = 0; u < B; ++u) {
        if (j0 + u < nv_lds) {
          stage[(j0 + u) * kStagedThreads + tid] = pack_bits<T, V>(pk[u]);
#pragma unroll
          for (int i = 0; i < V; ++i) sum += sl[u].ok ? to_f32(pk[u].v[i]) : 0.f;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < R; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) sum += rs[j].ok ? to_f32(reg[j].v[i]) : 0.f;
    }
    if (ragged) {  // the repeated elements of the last vector, off again
      const Pack<T, V> pk = bits_pack<T, V>(stage[j_tail * kStagedThreads + tid]);
#pragma unroll
      for (int i = 0; i < V - 1; ++i) sum -= i < lo_t ? to_f32(pk.v[i]) : 0.f;
    }
    const float mean = block_sum1(sum, red[0], NW) * inv_d;
    // ---- second pass over the staged row: squared deviations
    float m2 = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = rs[j].ok ? to_f32(reg[j].v[i]) - mean : 0.f;
        m2 += d * d;
      }
    }
    for (int j = 0; j < nv_lds; ++j) {
      const StagedSlot<V> sl = lds_slot(j);
      const Pack<T, V> pk = bits_pack<T, V>(stage[j * kStagedThreads + tid]);
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = sl.ok ? to_f32(pk.v[i]) - mean : 0.f;
        m2 += d * d;
      }
    }
    if (ragged) {
      const Pack<T, V> pk = bits_pack<T, V>(stage[j_tail * kStagedThreads + tid]);
#pragma unroll
      for (int i = 0; i < V - 1; ++i) {
        const float d = to_f32(pk.v[i]) - mean;
        m2 -= i < lo_t ? d * d : 0.f;
      }
    }
    const float rstd = rsqrtf(block_sum1(m2, red[1], NW) * inv_d + eps);
    if (tid == 0) {
      mean_out[row] = mean;
      rstd_out[row] = rstd;
    }
    // ---- normalise from the staged copy
    const int c = static_cast<int>(row % C);
    const float a = rstd * gamma[c], bs = beta[c];
    auto emit = [&](const Pack<T, V>& pk, const StagedSlot<V>& sl) {
      if (!sl.ok) return;
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) o.v[i] = from_f32<T>((to_f32(pk.v[i]) - mean) * a + bs);
      store_pack<T, V>(yr + sl.col, o);
    };
#pragma unroll
    for (int j = 0; j < R; ++j) emit(reg[j], rs[j]);
    for (int j = 0; j < nv_lds; ++j) emit(bits_pack<T, V>(stage[j * kStagedThreads + tid]), lds_slot(j));
    // (the next row's block sums reuse red[0] only after this row's second barrier)
  }
}

// Backward, channel-first InstanceNorm (gamma is the scalar of channel row % C): x and dy
// staged; the row sums a = sum dy, b = sum dy * xh go to part[n][0][c] = b, part[n][1][c] = a as
// in rows_bwd_resident.  dx may alias dy, not x.
template <typename T, int V>
__global__ void __launch_bounds__(kStagedThreads)
rows_bwd_staged(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
                const float* __restrict__ mean_in, const float* __restrict__ rstd_in, T* dx,
                float* __restrict__ part, int64_t n_rows, int d_elems, int C, int nv_lds) {
  constexpr int R = kStagedRegVec;
  constexpr int B = 4;
  constexpr int NW = kStagedThreads / kWave;
  __shared__ float2 red[2][16];
  extern __shared__ __attribute__((aligned(16))) unsigned char staged_bytes[];
  u32x4* stage = reinterpret_cast<u32x4*>(staged_bytes);  // [nv_lds][2][kStagedThreads]
  const int tid = static_cast<int>(threadIdx.x);
  const int64_t D = d_elems;
  const float inv_d = 1.0f / static_cast<float>(D);
  StagedSlot<V> rs[R];
#pragma unroll
  for (int j = 0; j < R; ++j) rs[j] = staged_slot<V>(tid + j * kStagedThreads, d_elems);
  auto lds_slot = [&](int j) { return staged_slot<V>(tid + (R + j) * kStagedThreads, d_elems); };
  // ragged rows: the LDS slot of the overlapping last vector and, in the thread that holds it,
  // the number of elements it repeats
  const bool ragged = d_elems % V != 0;
  const int j_tail = ragged ? (d_elems / V) / kStagedThreads - R : 0;
  const int lo_t = (ragged && tid == (d_elems / V) % kStagedThreads) ? V - d_elems % V : 0;

  int it = 0;
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x, ++it) {
    const T* xr = x + row * D;
    const T* dyr = dy + row * D;
    T* dxr = dx + row * D;
    const float mean = mean_in[row], rstd = rstd_in[row];
    const int c = static_cast<int>(row % C);
    const float gm = gamma[c];
    Pack<T, V> rx[R], rd[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
      rx[j] = load_pack_last<T, V>(xr + rs[j].col);
      rd[j] = load_pack_last<T, V>(dyr + rs[j].col);
    }
    float a1 = 0.f, a2 = 0.f;
    auto add = [&](const Pack<T, V>& px, const Pack<T, V>& pd, const StagedSlot<V>& sl) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float h = sl.ok ? (to_f32(px.v[i]) - mean) * rstd : 0.f;
        const float d = sl.ok ? to_f32(pd.v[i]) : 0.f;
        a1 += d;
        a2 += d * h;
      }
    };
    for (int j0 = 0; j0 < nv_lds; j0 += B) {
      Pack<T, V> px[B], pd[B];
      StagedSlot<V> sl[B];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        sl[u] = lds_slot(j0 + u < nv_lds ? j0 + u : nv_lds - 1);
        px[u] = load_pack_last<T, V>(xr + sl[u].col);
        pd[u] = load_pack_last<T, V>(dyr + sl[u].col);
      }
      batch_loaded<T, V, B>(px, pd);
#pragma unroll
      for (int u = 0; u < B; ++u) {
        if (j0 + u < nv_lds) {
          stage[((j0 + u) * 2 + 0) * kStagedThreads + tid] = pack_bits<T, V>(px[u]);
          stage[((j0 + u) * 2 + 1) * kStagedThreads + tid] = pack_bits<T, V>(pd[u]);
          add(px[u], pd[u], sl[u]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < R; ++j) add(rx[j], rd[j], rs[j]);
    if (ragged) {  // the repeated elements of the last vector, off again
      const Pack<T, V> px = bits_pack<T, V>(stage[(j_tail * 2 + 0) * kStagedThreads + tid]);
      const Pack<T, V> pd = bits_pack<T, V>(stage[(j_tail * 2 + 1) * kStagedThreads + tid]);
#pragma unroll
      for (int i = 0; i < V - 1; ++i) {
        const float h = (to_f32(px.v[i]) - mean) * rstd;
        const float d = to_f32(pd.v[i]);
        a1 -= i < lo_t ? d : 0.f;
        a2 -= i < lo_t ? d * h : 0.f;
      }
    }
    const float2 s = block_sum2(a1, a2, red[it & 1], NW);
    if (tid == 0) {
      const int64_t n = row / C;
      part[(n * 2 + 0) * C + c] = s.y;
      part[(n * 2 + 1) * C + c] = s.x;
    }
    const float scale = rstd * gm;
    const float ca = -scale * (s.y * inv_d), cb = -scale * (s.x * inv_d);
    auto emit = [&](const Pack<T, V>& px, const Pack<T, V>& pd, const StagedSlot<V>& sl) {
      if (!sl.ok) return;
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float h = (to_f32(px.v[i]) - mean) * rstd;
        o.v[i] = from_f32<T>(scale * to_f32(pd.v[i]) + (ca * h + cb));
      }
      store_pack<T, V>(dxr + sl.col, o);
    };
#pragma unroll
    for (int j = 0; j < R; ++j) emit(rx[j], rd[j], rs[j]);
    for (int j = 0; j < nv_lds; ++j) {
      emit(bits_pack<T, V>(stage[(j * 2 + 0) * kStagedThreads + tid]), bits_pack<T, V>(stage[(j * 2 + 1) * kStagedThreads + tid]),
           lds_slot(j));
    }
  }
}

// ------------------------------------------------------------- column reduction
// out0[j] = sum_g part[g][0][j], out1[j] = sum_g part[g][1][j] for j < W, g < G, summed
// in a fixed order (deterministic; the reference likewise uses no atomics,
// fused_layer_norm_op.cu:763-803, fused_instance_norm_op.cu:442-457).
// Block of 256 threads = CX column groups of CW floats x (256 / CX) slices of g; a block
// owns CX * CW adjacent columns of the concatenated [2W] row, so the grid has
// 2W / (CX * CW) blocks (128 for W = 1024).  Slices are folded by a lane butterfly and a
// 4-entry LDS step.
constexpr int kColReduceThreads = 256;

template <int CW, int CX>
__global__ void __launch_bounds__(kColReduceThreads)
col_reduce(const float* __restrict__ part, float* __restrict__ out0, float* __restrict__ out1,
           int G, int W, int64_t part_stride, int64_t out_stride) {
  // blockIdx.y: independent problems part + y * part_stride -> out + y * out_stride
  part += static_cast<int64_t>(blockIdx.y) * part_stride;
  out0 += static_cast<int64_t>(blockIdx.y) * out_stride;
  out1 += static_cast<int64_t>(blockIdx.y) * out_stride;
  // CX column groups of CW columns per block, CY = threads / CX partial rows in parallel:
  // CX = 4 for many partial rows, 64 for a few dozen, 256 (one thread per group, no
  // exchange) for a handful.
  constexpr int CY = kColReduceThreads / CX;
  constexpr int NW = kColReduceThreads / kWave;
  constexpr int HOLD = CX < kWave ? NW : CY;  // partial sums per column group after the wave fold
  __shared__ float buf[HOLD > 1 ? HOLD : 1][CX][CW];
  const int cx = threadIdx.x % CX;
  const int cy = threadIdx.x / CX;
  const int W2 = 2 * W;
  const int col = (blockIdx.x * CX + cx) * CW;  // column in the concatenated [2W] row
  float acc[CW];
#pragma unroll
  for (int i = 0; i < CW; ++i) acc[i] = 0.f;
  if (col < W2) {
    const float* p = part + col;
    int g = cy;
    for (; g + 3 * CY < G; g += 4 * CY) {
      float t0[CW], t1[CW], t2[CW], t3[CW];
      load_f32<CW>(p + static_cast<int64_t>(g) * W2, t0);
      load_f32<CW>(p + static_cast<int64_t>(g + CY) * W2, t1);
      load_f32<CW>(p + static_cast<int64_t>(g + 2 * CY) * W2, t2);
      load_f32<CW>(p + static_cast<int64_t>(g + 3 * CY) * W2, t3);
#pragma unroll
      for (int i = 0; i < CW; ++i) acc[i] += (t0[i] + t1[i]) + (t2[i] + t3[i]);
    }
    for (; g < G; g += CY) {
      float t[CW];
      load_f32<CW>(p + static_cast<int64_t>(g) * W2, t);
#pragma unroll
      for (int i = 0; i < CW; ++i) acc[i] += t[i];
    }
  }
  if constexpr (CX < kWave) {
    // lanes l, l + CX, ... of a wave hold slices of the same columns
#pragma unroll
    for (int i = 0; i < CW; ++i) {
#pragma unroll
      for (int m = CX; m < kWave; m <<= 1) acc[i] += lane_xor(acc[i], m);
    }
  }
  if constexpr (HOLD > 1) {
    const int lane = threadIdx.x & (kWave - 1);
    const int slot = CX < kWave ? threadIdx.x / kWave : cy;
    if (CX >= kWave || lane < CX) {
#pragma unroll
      for (int i = 0; i < CW; ++i) buf[slot][cx][i] = acc[i];
    }
    __syncthreads();
    if (threadIdx.x < CX) {
#pragma unroll
      for (int i = 0; i < CW; ++i) {
        float s = buf[0][cx][i];
#pragma unroll
        for (int k = 1; k < HOLD; ++k) s += buf[k][cx][i];
        acc[i] = s;
      }
    }
  }
  if (threadIdx.x < CX && col < W2) {
#pragma unroll
    for (int i = 0; i < CW; ++i) {
      // CW divides W on the vector path, so a column group never straddles the two halves
      const int j = col + i;
      if (j < W) {
        out0[j] = acc[i];
      } else if (j < W2) {
        out1[j - W] = acc[i];
      }
    }
  }
}

// ------------------------------------------------------------------------ split rows
// A row of D elements is cut into S chunks of `chunk` elements (the last may be short).
// Work item w = row * S + s; blocks take work items grid-stride.  V = elements per
// access (a 16-byte vector; a ragged row end is finished element-wise by one thread).
//
// Every loop over a chunk runs in batches of kSplitBatch accesses per thread whose loads are
// all issued before the first is consumed (a plain strided loop keeps one load per thread
// in flight, far too little to cover the memory latency at this bandwidth).  The second-
// stage kernels can walk their chunk backwards: stage 1 ends on the chunk's tail, so the
// tail is what the memory-side cache still holds when stage 2 starts.

constexpr int kSplitBatch = 4;
constexpr int kSplitThreads = 256;  // block size of every split_* launch

// Vector index of virtual position p of a chunk of n_vec vectors.
__device__ __forceinline__ int64_t split_pos(int64_t p, int64_t n_vec, bool rev) {
  return rev ? n_vec - 1 - p : p;
}

// Statistics of a chunk as a Welford triple.  Each thread takes its vectors in batches of
// kSplitBatch (all loads in flight), gets each batch's (mean, m2) from an exact two-pass over
// the registers and merges it into its running triple (wf_push); the block then merges the
// threads' triples with Chan's formula.  There is no pivot: no sample, however far from the
// rest, costs the others any precision.
template <typename T, int V>
__device__ __forceinline__ Wf chunk_wf(const T* p, int64_t len) {
  const int64_t n_vec = len / V;
  const int rem = static_cast<int>(len % V);  // only the last chunk of a ragged row
  const int64_t tid = threadIdx.x;
  const bool has_tail = rem != 0 && n_vec % kSplitThreads == tid;
  Wf w{0.f, 0.f, 0.f};
  batched_for<kSplitBatch>(
      tid, n_vec, kSplitThreads,
      [&](int64_t v, int64_t step) {
        Pack<T, V> pk[kSplitBatch];
#pragma unroll
        for (int u = 0; u < kSplitBatch; ++u) pk[u] = load_pack<T, V>(p + (v + u * step) * V);
        batch_loaded<T, V, kSplitBatch>(pk);
        float f[kSplitBatch * V];
#pragma unroll
        for (int u = 0; u < kSplitBatch; ++u) {
#pragma unroll
          for (int k = 0; k < V; ++k) f[u * V + k] = to_f32(pk[u].v[k]);
        }
        wf_push<kSplitBatch * V>(w, f);
      },
      [&](int64_t v) {
        const Pack<T, V> pk = load_pack<T, V>(p + v * V);
        float f[V];
#pragma unroll
        for (int k = 0; k < V; ++k) f[k] = to_f32(pk.v[k]);
        wf_push<V>(w, f);
      });
  if (has_tail) {
    for (int k = 0; k < rem; ++k) wf_push_batch(w, to_f32(p[n_vec * V + k]), 0.f, 1.f);
  }
  return w;
}

// stage 1 forward: stats[w] = (mean, m2) of chunk w; the count follows from geometry.
template <typename T, int V>
__global__ void __launch_bounds__(kSplitThreads) split_fwd_stats(const T* __restrict__ x, float2* __restrict__ stats,
                                int64_t n_rows, int64_t D, int S, int64_t chunk) {
  __shared__ Wf wf_buf[2][16];
  const int64_t n_work = n_rows * S;
  int it = 0;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x, ++it) {
    const int64_t row = w / S;
    const int s = static_cast<int>(w % S);
    const int64_t beg = static_cast<int64_t>(s) * chunk;
    const int64_t len = (beg + chunk <= D ? chunk : D - beg);
    Wf r = chunk_wf<T, V>(x + row * D + beg, len);
    r = block_wf(r, wf_buf[it & 1], kSplitThreads / kWave);
    if (threadIdx.x == 0) stats[w] = make_float2(r.mean, r.m2);
  }
}

// Statistics of a row from those of its S chunks (S <= 1024), the same in every lane of every
// wave: lane l takes chunks l, l + 64, ... (all its loads in flight at once), and the row is
//     mean = sum_s n_s mean_s / D,      m2 = sum_s [ m2_s + n_s (mean_s - mean)^2 ]
// which is Chan's merge (norm_util.h:190-210) of all chunks at once: every term of m2 is
// non-negative and there is no chain of S dependent merges.  The sums over the lanes are
// commutative butterflies, so every workgroup of the row gets the same bits.
__device__ __forceinline__ Wf merge_chunks(const float2* stats, int S, int64_t D, int64_t chunk) {
#pragma clang fp contract(off)
  constexpr int B = 4;
  const int lane = static_cast<int>(threadIdx.x) & (kWave - 1);
  const float n_full = static_cast<float>(chunk);
  const float n_last = static_cast<float>(D - static_cast<int64_t>(S - 1) * chunk);
  const float inv_d = 1.0f / static_cast<float>(D);
  auto count = [&](int k) { return k >= S ? 0.f : (k == S - 1 ? n_last : n_full); };
  float s1 = 0.f, m2 = 0.f, mean;
  if (S <= B * kWave) {  // one round trip
    float2 t[B];
#pragma unroll
    for (int u = 0; u < B; ++u) {
      const int k = lane + u * kWave;
      t[u] = stats[k < S ? k : 0];
    }
#pragma unroll
    for (int u = 0; u < B; ++u) s1 += t[u].x * count(lane + u * kWave);
    mean = group_sum<kWave>(s1) * inv_d;
#pragma unroll
    for (int u = 0; u < B; ++u) {
      const float n = count(lane + u * kWave);
      const float d = t[u].x - mean;
      m2 += n == 0.f ? 0.f : t[u].y + n * (d * d);
    }
  } else {
    for (int k0 = lane; k0 < S; k0 += B * kWave) {
      float2 t[B];
#pragma unroll
      for (int u = 0; u < B; ++u) t[u] = stats[k0 + u * kWave < S ? k0 + u * kWave : 0];
#pragma unroll
      for (int u = 0; u < B; ++u) s1 += t[u].x * count(k0 + u * kWave);
    }
    mean = group_sum<kWave>(s1) * inv_d;
    for (int k0 = lane; k0 < S; k0 += B * kWave) {
      float2 t[B];
#pragma unroll
      for (int u = 0; u < B; ++u) t[u] = stats[k0 + u * kWave < S ? k0 + u * kWave : 0];
#pragma unroll
      for (int u = 0; u < B; ++u) {
        const float n = count(k0 + u * kWave);
        const float d = t[u].x - mean;
        m2 += n == 0.f ? 0.f : t[u].y + n * (d * d);
      }
    }
  }
  m2 = group_sum<kWave>(m2);
  return Wf{mean, m2, static_cast<float>(D)};
}

// Sums of a row from those of its S chunks, likewise in every lane of every wave.
__device__ __forceinline__ float2 sum_chunks(const float2* sums, int S) {
  constexpr int B = 4;
  const int lane = static_cast<int>(threadIdx.x) & (kWave - 1);
  float a = 0.f, b = 0.f;
  for (int k0 = lane; k0 < S; k0 += B * kWave) {
    float2 t[B];
#pragma unroll
    for (int u = 0; u < B; ++u) t[u] = sums[k0 + u * kWave < S ? k0 + u * kWave : 0];
#pragma unroll
    for (int u = 0; u < B; ++u) {
      a += k0 + u * kWave < S ? t[u].x : 0.f;
      b += k0 + u * kWave < S ? t[u].y : 0.f;
    }
  }
  return make_float2(group_sum<kWave>(a), group_sum<kWave>(b));
}

// stage 2 forward: merge the S chunk statistics of the row, normalise the chunk.
// y may alias x: stage 1 has completed (it is an earlier launch on the same stream) and
// every thread reads its vectors of a batch before it writes the same vectors.
template <typename T, int V, bool ROW_AFFINE>
__global__ void __launch_bounds__(kSplitThreads) split_fwd_apply(const T* x, const float2* __restrict__ stats,
                                const float* __restrict__ gamma, const float* __restrict__ beta,
                                T* y, float* __restrict__ mean_out,
                                float* __restrict__ rstd_out, int64_t n_rows, int64_t D, int S,
                                int64_t chunk, int C, float eps, int rev) {
  constexpr int B = ROW_AFFINE ? kSplitBatch : 2;  // the per-column gamma / beta take registers
  const int64_t n_work = n_rows * S;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const int64_t row = w / S;
    const int s = static_cast<int>(w % S);
    const Wf r = merge_chunks(stats + row * S, S, D, chunk);
    const float mean = r.mean;
    const float rstd = rsqrtf(r.m2 / static_cast<float>(D) + eps);
    if (s == 0 && threadIdx.x == 0) {
      mean_out[row] = mean;
      rstd_out[row] = rstd;
    }
    float gs = 1.f, bs = 0.f;
    if constexpr (ROW_AFFINE) {
      const int c = static_cast<int>(row % C);
      gs = gamma[c];
      bs = beta[c];
    }
    const int64_t beg = static_cast<int64_t>(s) * chunk;
    const int64_t len = (beg + chunk <= D ? chunk : D - beg);
    const int64_t n_vec = len / V;
    const T* xp = x + row * D + beg;
    T* yp = y + row * D + beg;
    const float* gp = gamma + beg;
    const float* bp = beta + beg;
    const float a = rstd * gs;  // ROW_AFFINE: y = (x - mean) * a + bs
    auto one = [&](const Pack<T, V>& pk, int64_t i) {
      Pack<T, V> o;
      if constexpr (ROW_AFFINE) {
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = from_f32<T>((to_f32(pk.v[k]) - mean) * a + bs);
      } else {
        float tg[V], tb[V];
        load_f32<V>(gp + i, tg);
        load_f32<V>(bp + i, tb);
#pragma unroll
        for (int k = 0; k < V; ++k) {
          o.v[k] = from_f32<T>((to_f32(pk.v[k]) - mean) * rstd * tg[k] + tb[k]);
        }
      }
      store_pack<T, V>(yp + i, o);
    };
    batched_for<B>(
        threadIdx.x, n_vec, kSplitThreads,
        [&](int64_t v, int64_t step) {
          Pack<T, V> pk[B];
          int64_t i[B];
#pragma unroll
          for (int u = 0; u < B; ++u) {
            i[u] = split_pos(v + u * step, n_vec, rev) * V;
            pk[u] = load_pack_last<T, V>(xp + i[u]);
          }
          batch_loaded<T, V, B>(pk);
#pragma unroll
          for (int u = 0; u < B; ++u) one(pk[u], i[u]);
        },
        [&](int64_t v) {
          const int64_t i = split_pos(v, n_vec, rev) * V;
          one(load_pack_last<T, V>(xp + i), i);
        });
    // ragged row end (last chunk only): the elements after the last full vector
    const int rem = static_cast<int>(len % V);
    if (rem != 0 && n_vec % kSplitThreads == threadIdx.x) {
      const int64_t i = n_vec * V;
      Pack<T, V> o;
      const Pack<T, V> pk = load_pack_n<T, V>(xp + i, rem);
      if constexpr (ROW_AFFINE) {
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = from_f32<T>((to_f32(pk.v[k]) - mean) * a + bs);
      } else {
        float tg[V], tb[V];
        load_f32_n<V>(gp + i, tg, rem);
        load_f32_n<V>(bp + i, tb, rem);
#pragma unroll
        for (int k = 0; k < V; ++k) o.v[k] = from_f32<T>((to_f32(pk.v[k]) - mean) * rstd * tg[k] + tb[k]);
      }
      store_pack_n<T, V>(yp + i, o, rem);
    }
  }
}

// stage 1 backward: sums[w] = (sum g, sum g * xh) over chunk w, g = dy * gamma
// (ROW_AFFINE: (sum dy, sum dy * xh), gamma applied in stage 2).
template <typename T, int V, bool ROW_AFFINE>
__global__ void __launch_bounds__(kSplitThreads) split_bwd_sums(const T* __restrict__ dy, const T* __restrict__ x,
                               const float* __restrict__ gamma,
                               const float* __restrict__ mean_in,
                               const float* __restrict__ rstd_in, float2* __restrict__ sums,
                               int64_t n_rows, int64_t D, int S, int64_t chunk) {
  constexpr int B = ROW_AFFINE ? kSplitBatch : 2;
  __shared__ float2 sum_buf[2][16];
  const int64_t n_work = n_rows * S;
  int it = 0;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x, ++it) {
    const int64_t row = w / S;
    const int s = static_cast<int>(w % S);
    const int64_t beg = static_cast<int64_t>(s) * chunk;
    const int64_t len = (beg + chunk <= D ? chunk : D - beg);
    const int64_t n_vec = len / V;
    const float mean = mean_in[row], rstd = rstd_in[row];
    const T* xp = x + row * D + beg;
    const T* dp = dy + row * D + beg;
    const float* gp = gamma + beg;
    // accumulate sum g and sum g * x; sum g * xh = rstd * (sum g * x - mean * sum g)
    // would cancel for |mean| >> 1 / rstd, so x is centred first (one subtraction)
    float s1 = 0.f, s2 = 0.f;
    auto one = [&](const Pack<T, V>& px, const Pack<T, V>& pd, int64_t i) {
      float tg[V];
      if constexpr (!ROW_AFFINE) load_f32<V>(gp + i, tg);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const float xc = to_f32(px.v[k]) - mean;
        float gv = to_f32(pd.v[k]);
        if constexpr (!ROW_AFFINE) gv *= tg[k];
        s1 += gv;
        s2 += gv * xc;
      }
    };
    batched_for<B>(
        threadIdx.x, n_vec, kSplitThreads,
        [&](int64_t v, int64_t step) {
          Pack<T, V> px[B], pd[B];
#pragma unroll
          for (int u = 0; u < B; ++u) {
            px[u] = load_pack<T, V>(xp + (v + u * step) * V);
            pd[u] = load_pack<T, V>(dp + (v + u * step) * V);
          }
          batch_loaded<T, V, B>(px, pd);
#pragma unroll
          for (int u = 0; u < B; ++u) one(px[u], pd[u], (v + u * step) * V);
        },
        [&](int64_t v) { one(load_pack<T, V>(xp + v * V), load_pack<T, V>(dp + v * V), v * V); });
    const int rem = static_cast<int>(len % V);
    if (rem != 0 && n_vec % kSplitThreads == threadIdx.x) {
      // zero-filled dy beyond the row end adds nothing
      const int64_t i = n_vec * V;
      const Pack<T, V> px = load_pack_n<T, V>(xp + i, rem);
      const Pack<T, V> pd = load_pack_n<T, V>(dp + i, rem);
      float tg[V];
      if constexpr (!ROW_AFFINE) load_f32_n<V>(gp + i, tg, rem);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        const float xc = to_f32(px.v[k]) - mean;
        float gv = to_f32(pd.v[k]);
        if constexpr (!ROW_AFFINE) gv *= tg[k];
        s1 += gv;
        s2 += gv * xc;
      }
    }
    const float2 r = block_sum2(s1, s2 * rstd, sum_buf[it & 1], kSplitThreads / kWave);
    if (threadIdx.x == 0) sums[w] = r;
  }
}

// stage 2 backward: merge the row's chunk sums, write dx for the chunk.  ROW_AFFINE also
// writes the per-(n, c) sums into `part` (layout as in rows_bwd_resident).
template <typename T, int V, bool ROW_AFFINE>
__global__ void __launch_bounds__(kSplitThreads) split_bwd_apply(const T* dy, const T* __restrict__ x,
                                const float* __restrict__ gamma,
                                const float* __restrict__ mean_in,
                                const float* __restrict__ rstd_in,
                                const float2* __restrict__ sums, T* dx,
                                float* __restrict__ part, int64_t n_rows, int64_t D, int S,
                                int64_t chunk, int C, int rev) {
  constexpr int B = ROW_AFFINE ? kSplitBatch : 2;
  const int64_t n_work = n_rows * S;
  const float inv_d = 1.0f / static_cast<float>(D);
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const int64_t row = w / S;
    const int s = static_cast<int>(w % S);
    const float2 st = sum_chunks(sums + row * S, S);
    const float s1 = st.x, s2 = st.y;
    const float mean = mean_in[row], rstd = rstd_in[row];
    float gs = 1.f;
    if constexpr (ROW_AFFINE) {
      const int64_t n = row / C;
      const int c = static_cast<int>(row % C);
      gs = gamma[c];
      if (s == 0 && threadIdx.x == 0) {
        part[(n * 2 + 0) * C + c] = s2;
        part[(n * 2 + 1) * C + c] = s1;
      }
    }
    const int64_t beg = static_cast<int64_t>(s) * chunk;
    const int64_t len = (beg + chunk <= D ? chunk : D - beg);
    const int64_t n_vec = len / V;
    const T* xp = x + row * D + beg;
    const T* dp = dy + row * D + beg;
    T* op = dx + row * D + beg;
    const float* gp = gamma + beg;
    // dx = rstd * gs * (g - s1 / D - xh * s2 / D) = ca * g + cb * (x - mean) + cc
    const float ca = rstd * gs;
    const float cb = -ca * s2 * inv_d * rstd;
    const float cc = -ca * s1 * inv_d;
    auto one = [&](const Pack<T, V>& px, const Pack<T, V>& pd, int64_t i) {
      Pack<T, V> o;
      float tg[V];
      if constexpr (!ROW_AFFINE) load_f32<V>(gp + i, tg);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        float gv = to_f32(pd.v[k]);
        if constexpr (!ROW_AFFINE) gv *= tg[k];
        o.v[k] = from_f32<T>(ca * gv + (cb * (to_f32(px.v[k]) - mean) + cc));
      }
      store_pack<T, V>(op + i, o);
    };
    batched_for<B>(
        threadIdx.x, n_vec, kSplitThreads,
        [&](int64_t v, int64_t step) {
          Pack<T, V> px[B], pd[B];
          int64_t i[B];
#pragma unroll
          for (int u = 0; u < B; ++u) {
            i[u] = split_pos(v + u * step, n_vec, rev) * V;
            px[u] = load_pack_last<T, V>(xp + i[u]);
            pd[u] = load_pack_last<T, V>(dp + i[u]);
          }
          batch_loaded<T, V, B>(px, pd);
#pragma unroll
          for (int u = 0; u < B; ++u) one(px[u], pd[u], i[u]);
        },
        [&](int64_t v) {
          const int64_t i = split_pos(v, n_vec, rev) * V;
          one(load_pack_last<T, V>(xp + i), load_pack_last<T, V>(dp + i), i);
        });
    const int rem = static_cast<int>(len % V);
    if (rem != 0 && n_vec % kSplitThreads == threadIdx.x) {
      const int64_t i = n_vec * V;
      const Pack<T, V> px = load_pack_n<T, V>(xp + i, rem);
      const Pack<T, V> pd = load_pack_n<T, V>(dp + i, rem);
      Pack<T, V> o;
      float tg[V];
      if constexpr (!ROW_AFFINE) load_f32_n<V>(gp + i, tg, rem);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        float gv = to_f32(pd.v[k]);
        if constexpr (!ROW_AFFINE) gv *= tg[k];
        o.v[k] = from_f32<T>(ca * gv + (cb * (to_f32(px.v[k]) - mean) + cc));
      }
      store_pack_n<T, V>(op + i, o, rem);
    }
  }
}

}  // namespace atexn
