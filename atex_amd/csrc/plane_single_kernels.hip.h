// Channel-first InstanceNorm planes that do not fit one workgroup, in ONE launch per direction
// and ONE pass over the data.
//
// The two-stage kernels (split_* in rows_kernels.hip.h) read x (and dy) twice: once for the
// statistics of a plane, once to apply them.  Here a plane of D elements is cut into S chunks of
// at most 8 vectors per thread of a 512-thread workgroup, every chunk stays in its workgroup's
// registers, and the S workgroups of a plane exchange their chunk statistics through memory
// while they run (the tagged pairs of norm_common.hip.h: a value and the call's tag in one
// 8-byte word, no flag, no fence, nothing to clear):
//
//   1. every workgroup loads its chunk, computes the chunk's (mean, m2) [backward: the two
//      sums] and publishes them as one tagged pair;
//   2. wave 0 of every workgroup waits, a lane per chunk, for the S pairs of its plane and
//      merges them (every workgroup of the plane computes the same bits);
//   3. the workgroup applies the plane's statistics to the chunk it still holds and stores it.
//
// A launch has many more workgroups than the chip holds at once; what the exchange needs is only
// that the S workgroups of ONE plane are resident together, on one XCD (plain stores then reach
// the L2 that the device-scope polls read).  The grid is laid out for that: workgroups are dealt
// to the 8 XCDs in turn (workgroup b runs on XCD b % 8) and each XCD starts its workgroups in
// index order, so workgroup b takes chunk (b / 8) % S of plane ((b / 8) / S) * 8 + b % 8: the
// planes of an XCD follow one another, each as S consecutive workgroups of that XCD, and a
// workgroup only ever waits for workgroups that were started before or together with it.  The
// host takes this path when S is at most the number of such workgroups an XCD holds (two per CU).
//
// Nothing here can hang: every wait is a bounded number of polls.  A workgroup whose wait runs
// out (its peers are not resident: another kernel holds the CUs; or the placement assumption
// does not hold on this device) computes, with the same code and therefore to the same bits,
// the pairs that have not arrived from x (and dy) itself, and publishes them: whoever gives up
// first does the missing chunks for everybody.  That is why the host keeps callers that pass
// y == x (dx == dy) on the two-stage kernels: a peer may already have overwritten its chunk by
// then.
//
// Counterpart in the reference: the two-kernel channel-first path for large planes
// (fused_instance_norm_op.cu:1311-1455 forward, 1168-1309 backward), which reads its inputs
// twice.
#pragma once

#include "norm_common.hip.h"

namespace atexn {

constexpr int kPlaneThreads = 512;    // threads of a workgroup
constexpr int kPlaneMaxChunks = 64;   // chunks per plane: a lane each in the merge
constexpr int kPlaneXcds = 8;

struct PlaneGeom {
  int64_t row;    // plane (n * C + c)
  int s;          // chunk of the plane
  bool active;    // the grid is padded to a whole number of planes per XCD
};
__device__ __forceinline__ PlaneGeom plane_geom(int64_t n_rows, int S) {
  const unsigned b = blockIdx.x;
  const unsigned xcd = b % kPlaneXcds, j = b / kPlaneXcds;
  PlaneGeom g;
  g.row = static_cast<int64_t>(j / static_cast<unsigned>(S)) * kPlaneXcds + xcd;
  g.s = static_cast<int>(j % static_cast<unsigned>(S));
  g.active = g.row < n_rows;
  return g;
}

// Chunk l of a plane of n_vec vectors: vectors [l * chunk_vec, l * chunk_vec + n_here).
__device__ __forceinline__ int plane_chunk_vectors(int l, int S, int n_vec, int chunk_vec) {
  return l == S - 1 ? n_vec - (S - 1) * chunk_vec : chunk_vec;
}

// Thread t holds vectors t, t + 512, ... of the chunk at p (n_here vectors); FULL: every thread
// holds U of them.  A vector outside the chunk is not loaded and reads as zeros.  NT: loads with
// the non-temporal hint.  The data is read once, so the backward always uses it ([2, 32, 128^3]
// fp16 150.5 -> 146.0 us, [16, 64, 256, 256] 73.9 -> 70.6 us).  The forward gains as much on
// tensors that no cache level can retain (268 MB: 95.0 -> 91.8 us) but loses on smaller ones when
// the same x comes round again before the memory-side cache has let go of it (134 MB per tensor,
// three buffer sets in rotation: 40 -> 47 us whatever the number of chunks): the host asks for it
// from 256 MiB.
// AGAIN: a load on a path that is seldom taken computes its addresses there, from a thread
// index that the compiler treats as a new value, instead of keeping the addresses of the kernel's
// first load alive all the way through the common path.
template <typename T, int V, int U, bool FULL, bool NT, bool AGAIN = false>
__device__ __forceinline__ void plane_load(const T* p, int n_here, Pack<T, V> (&raw)[U]) {
  unsigned tid = threadIdx.x;
  if constexpr (AGAIN) asm volatile("" : "+v"(tid));
#pragma unroll
  for (int k = 0; k < U; ++k) {
    // (a 32-bit element offset from the chunk's start, which is the same for the whole workgroup)
    const unsigned i = tid + static_cast<unsigned>(k * kPlaneThreads);
    const T* q = p + i * static_cast<unsigned>(V);
    if constexpr (FULL) {
      raw[k] = NT ? load_pack_last<T, V>(q) : load_pack<T, V>(q);
    } else {
      __builtin_memset(&raw[k], 0, sizeof(raw[k]));
      if (i < static_cast<unsigned>(n_here)) raw[k] = NT ? load_pack_last<T, V>(q) : load_pack<T, V>(q);
    }
  }
}
// how many of a thread's U vectors lie inside the chunk (they are the first ones)
template <int U, bool FULL>
__device__ __forceinline__ int plane_valid(int n_here) {
  if (FULL) return U;
  const int left = n_here - static_cast<int>(threadIdx.x);
  const int n = (left + kPlaneThreads - 1) / kPlaneThreads;
  return left <= 0 ? 0 : (n < U ? n : U);
}

// (mean, m2) of the chunk held in raw: exact two-pass per thread over its registers, Chan's merge
// over the workgroup.  The same in every thread.
template <typename T, int V, int U, bool FULL>
__device__ __forceinline__ Wf plane_chunk_stats(Pack<T, V> (&raw)[U], int n_here, Wf* buf) {
  Wf w;
  if constexpr (FULL) {
    // wf_push over the thread's U * V elements, written out so that the second pass converts
    // the elements again rather than keeping U * V floats alive beside the raw vectors (bf16
    // has no mixed-precision arithmetic that would take the raw halves as they are: it came to
    // 109 registers, or 98 spilled ones under the bound of 64)
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < U; ++k) {
#pragma unroll
      for (int i = 0; i < V; ++i) s += to_f32(raw[k].v[i]);
    }
    const float mb = s * (1.0f / (U * V));
#pragma unroll
    for (int k = 0; k < U; ++k) forget_derived(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < U; ++k) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = to_f32(raw[k].v[i]) - mb;
        q += d * d;
      }
    }
    w = Wf{0.f, 0.f, 0.f};
    wf_push_batch(w, mb, q, static_cast<float>(U * V));
  } else {
    // the thread's first nv vectors are inside the chunk
    const int nv = plane_valid<U, FULL>(n_here);
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < U; ++k) {
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < V; ++i) t += to_f32(raw[k].v[i]);
      s += k < nv ? t : 0.f;
    }
    w.n = static_cast<float>(nv * V);
    w.mean = nv > 0 ? s / w.n : 0.f;
    // (the second pass converts the elements again rather than keeping 64 floats alive)
#pragma unroll
    for (int k = 0; k < U; ++k) forget_derived(raw[k]);
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < U; ++k) {
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float d = to_f32(raw[k].v[i]) - w.mean;
        t += d * d;
      }
      q += k < nv ? t : 0.f;
    }
    w.m2 = q;
  }
  return block_wf(w, buf, kPlaneThreads / kWave);
}

// (mean, m2) of a plane from its chunks' (mean, m2), one chunk per lane of a wave (lanes >= S
// hold nothing): Chan's merge of all chunks at once, every term of m2 non-negative.
__device__ __forceinline__ void plane_merge_stats(float pm, float pq, int lane, int S, float n_full, float n_last,
                                                  float inv_d, float& mean, float& m2) {
#pragma clang fp contract(off)
  const bool in = lane < S;
  const float w = lane == S - 1 ? n_last : n_full;
  mean = group_sum<kWave>(in ? pm * w : 0.f) * inv_d;
  const float d = pm - mean;
  m2 = group_sum<kWave>(in ? pq + w * (d * d) : 0.f);
}

// A workgroup's fallback (its wait for the pairs of a plane has run out): the chunks whose pairs
// are missing get computed, each once, by the workgroups that have given up.  Round by round a
// workgroup looks, a lane per chunk, at what has arrived (plane_look), claims ONE missing chunk
// that nobody has claimed yet (a compare-and-swap on the chunk's claim word: the call's tag),
// computes its pair as the chunk's own workgroup would, publishes it, and looks again; when
// nothing is left to claim, whatever is still missing is in the hands of a running workgroup
// and only has to be waited for.  (When the workgroups of a plane cannot be resident together
// because another kernel fills part of the chip, the resident ones thus share out the chunks of
// the absent ones instead of each redoing the whole plane; the absent ones, once started, find
// their pairs published, publish them again with the same bits and go on.)
__device__ __forceinline__ void plane_look(const cl_word* pairs, int S, unsigned tag, int (&have)[kPlaneMaxChunks]) {
  __syncthreads();  // whatever read have before is done
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    bool ok = false;
    if (lane < S) {
      const cl_word w0 = cl_peek(pairs + 2 * lane);
      const cl_word w1 = cl_peek(pairs + 2 * lane + 1);
      ok = static_cast<unsigned>(w0 >> 32) == tag && static_cast<unsigned>(w1 >> 32) == ~tag;
    }
    have[lane] = ok ? 1 : 0;
  }
  __syncthreads();
}
__device__ __forceinline__ bool plane_try_claim(unsigned* word, unsigned tag) {
  unsigned cur = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (cur == tag) return false;
  return __hip_atomic_compare_exchange_strong(word, &cur, tag, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
}
// compute(l) returns the pair of chunk l in every thread (it contains barriers and is called by
// the whole workgroup).  s_self: where this workgroup starts looking for a chunk to claim.
template <typename F>
__device__ __forceinline__ void plane_fill_missing(cl_word* pairs, unsigned* claims, int S, int s_self, unsigned tag,
                                                   int (&have)[kPlaneMaxChunks], F&& compute) {
  __shared__ int sm_pick;
  for (int round = 0; round < S; ++round) {
    plane_look(pairs, S, tag, have);
    if (threadIdx.x == 0) {
      int pick = -1;
      for (int i = 1; i <= S && pick < 0; ++i) {
        const int l = (s_self + i) % S;
        if (!have[l] && plane_try_claim(claims + l, tag)) pick = l;
      }
      sm_pick = pick;
    }
    __syncthreads();
    const int l = sm_pick;
    if (l < 0) break;  // uniform
    const float2 t = compute(l);
    if (threadIdx.x == 0) cl_publish(pairs + 2 * l, t.x, t.y, tag);
  }
}
// Polls that a workgroup allows for pairs that are in the hands of running workgroups (or its
// own) to show up: they are on their way, this only bounds the wait.  Should they not show up
// after all, the result is marked (NaN) rather than computed from whatever the words held.
constexpr int kPlaneOwnPolls = 1 << 16;
__device__ __forceinline__ void plane_wait_own(const cl_word* pair, bool want, unsigned tag, float& a, float& b) {
  if (!cl_wait_pair(pair, want, tag, kPlaneOwnPolls, a, b)) a = b = __builtin_nanf("");
}

// ------------------------------------------------------------------------------ forward
// tagged: [n_rows][S] pairs (mean, m2) of the chunks.  n_vec = D / V, chunk_vec <= U * 512.
// (FULL: built for four workgroups per CU, 64 VGPRs, which the path that every launch takes needs
// anyway; the fallback then keeps a few values in scratch memory)
template <typename T, int V, int U, bool FULL, bool NT>
__global__ void __launch_bounds__(kPlaneThreads, FULL ? (__is_same(T, bf16_t) ? 6 : 8) : 4)
plane_fwd_single(const T* __restrict__ x, cl_word* tagged, unsigned* claims, const float* __restrict__ gamma,
                 const float* __restrict__ beta, T* __restrict__ y, float* __restrict__ mean_out,
                 float* __restrict__ rstd_out, int64_t n_rows, int n_vec, int S, int chunk_vec, int C, float eps,
                 unsigned tag, int max_polls, unsigned* trouble) {
  __shared__ Wf wf_buf[2][16];
  __shared__ int have[kPlaneMaxChunks];
  __shared__ float sm_mean, sm_rstd;
  __shared__ int sm_fail;
  const PlaneGeom g = plane_geom(n_rows, S);
  if (!g.active) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t D = static_cast<int64_t>(n_vec) * V;
  const T* xr = x + g.row * D;
  const int n_here = plane_chunk_vectors(g.s, S, n_vec, chunk_vec);
  const float n_full = static_cast<float>(chunk_vec) * V;
  const float n_last = static_cast<float>(plane_chunk_vectors(S - 1, S, n_vec, chunk_vec)) * V;
  const float inv_d = 1.0f / static_cast<float>(D);
  Pack<T, V> raw[U];
  plane_load<T, V, U, FULL, NT>(xr + static_cast<int64_t>(g.s) * chunk_vec * V, n_here, raw);
  const int c = static_cast<int>(g.row % C);
  const float gm = gamma[c], bt = beta[c];
  if (threadIdx.x == 0) sm_fail = 0;
  const Wf mine = plane_chunk_stats<T, V, U, FULL>(raw, n_here, wf_buf[0]);
  if (threadIdx.x == 0) cl_publish(tagged + (g.row * S + g.s) * 2, mine.mean, mine.m2, tag);
#pragma unroll
  for (int k = 0; k < U; ++k) forget_derived(raw[k]);
  if (wave == 0) {
    float pm, pq;
    if (exchange_wait_pair(tagged + (g.row * S + (lane < S ? lane : 0)) * 2, lane < S, tag, max_polls, trouble, pm, pq)) {
      float mu, q;
      plane_merge_stats(pm, pq, lane, S, n_full, n_last, inv_d, mu, q);
      if (lane == 0) {
        sm_mean = mu;
        sm_rstd = rsqrtf(__builtin_fmaf(q, inv_d, eps));
      }
    } else if (lane == 0) {
      sm_fail = 1;
    }
  }
  __syncthreads();
  if (sm_fail) {
    // See plane_fill_missing.  The chunks pass through the registers of the workgroup's own
    // chunk, which is loaded again at the end (x is intact: y != x).
    int it = 1;
    plane_fill_missing(tagged + g.row * S * 2, claims + g.row * S, S, g.s, tag, have, [&](int l) {
      const int n_l = plane_chunk_vectors(l, S, n_vec, chunk_vec);
      plane_load<T, V, U, FULL, NT>(xr + static_cast<int64_t>(l) * chunk_vec * V, n_l, raw);
      const Wf w = plane_chunk_stats<T, V, U, FULL>(raw, n_l, wf_buf[it++ & 1]);
      return make_float2(w.mean, w.m2);
    });
    if (wave == 0) {
      float pm, pq, mu, q;
      plane_wait_own(tagged + (g.row * S + (lane < S ? lane : 0)) * 2, lane < S, tag, pm, pq);
      plane_merge_stats(pm, pq, lane, S, n_full, n_last, inv_d, mu, q);
      if (lane == 0) {
        sm_mean = mu;
        sm_rstd = rsqrtf(__builtin_fmaf(q, inv_d, eps));
      }
    }
    plane_load<T, V, U, FULL, NT, true>(xr + static_cast<int64_t>(g.s) * chunk_vec * V, n_here, raw);
    __syncthreads();
  }
  const float mean = sm_mean, rstd = sm_rstd;
  if (g.s == 0 && threadIdx.x == 0) {
    mean_out[g.row] = mean;
    rstd_out[g.row] = rstd;
  }
  const float a = rstd * gm;  // y = (x - mean) * a + bt
  T* yr = y + g.row * D + static_cast<int64_t>(g.s) * chunk_vec * V;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = static_cast<int>(threadIdx.x) + k * kPlaneThreads;
    if (FULL || i < n_here) {
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) o.v[e] = from_f32<T>((to_f32(raw[k].v[e]) - mean) * a + bt);
      store_pack<T, V>(yr + static_cast<int64_t>(i) * V, o);
    }
  }
}

// ----------------------------------------------------------------------------- backward
// (sum dy, sum dy * xh) of the chunk held in rx / rd, the same in every thread.
template <typename T, int V, int U, bool FULL>
__device__ __forceinline__ float2 plane_chunk_sums(const Pack<T, V> (&rx)[U], const Pack<T, V> (&rd)[U], int n_here,
                                                   float mean, float rstd, float2* buf) {
  float s1 = 0.f, s2 = 0.f;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const bool in = FULL || static_cast<int>(threadIdx.x) + k * kPlaneThreads < n_here;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      // x is centred before the product: sum dy * x - mean * sum dy would cancel for |mean| >> 1 / rstd
      const float d = in ? to_f32(rd[k].v[i]) : 0.f;
      const float xc = to_f32(rx[k].v[i]) - mean;
      s1 += d;
      s2 += d * xc;
    }
  }
  return block_sum2(s1, s2 * rstd, buf, kPlaneThreads / kWave);
}

// (sum dy, sum dy * xh) of a whole plane when the wait for its chunks' pairs has run out: what is
// missing gets computed (plane_fill_missing; the chunks pass through rx / rd, the caller reloads
// its own afterwards), then the pairs are added up as the gathering wave adds them.  The result
// is valid in wave 0; contains barriers.
template <typename T, int V, int U, bool FULL>
__device__ __forceinline__ float2 plane_sums_alone(const T* xr, const T* dr, float mean, float rstd, int S, int s_self,
                                                   int n_vec, int chunk_vec, Pack<T, V> (&rx)[U], Pack<T, V> (&rd)[U],
                                                   float2 (&sum_buf)[2][16], int (&have)[kPlaneMaxChunks],
                                                   cl_word* pairs, unsigned* claims, unsigned tag) {
  const int lane = threadIdx.x & (kWave - 1);
  int it = 0;
  plane_fill_missing(pairs, claims, S, s_self, tag, have, [&](int l) {
    const int n_l = plane_chunk_vectors(l, S, n_vec, chunk_vec);
    const int64_t o = static_cast<int64_t>(l) * chunk_vec * V;
    plane_load<T, V, U, FULL, true>(xr + o, n_l, rx);
    plane_load<T, V, U, FULL, true>(dr + o, n_l, rd);
    return plane_chunk_sums<T, V, U, FULL>(rx, rd, n_l, mean, rstd, sum_buf[it++ & 1]);
  });
  float pa = 0.f, pb = 0.f;
  if (threadIdx.x < kWave) plane_wait_own(pairs + 2 * (lane < S ? lane : 0), lane < S, tag, pa, pb);
  const float a = group_sum<kWave>(lane < S ? pa : 0.f);
  const float b = group_sum<kWave>(lane < S ? pb : 0.f);
  return make_float2(a, b);
}

// The fold of the planes' sums over the batch inside plane_bwd_single (instead of a col_reduce
// launch after it): the workgroup of chunk 0 of every plane publishes the plane's sums as a
// tagged pair, and the one of the LAST instance's plane of channel c waits for the N pairs of c,
// a lane per instance, after it has stored its dx.  With C a multiple of the XCD count the planes
// of a channel run on one XCD, the last instance's after the others.  tagged == nullptr: the
// sums go to `part` for a col_reduce launch.
struct PlaneFold {
  cl_word* tagged;  // [n_rows] pairs (sum dy * xh, sum dy)
  float* dgamma;
  float* dbeta;
  int N;  // instances, 1 <= N <= 64
};

// tagged: [n_rows][S] pairs (sum dy, sum dy * xh) of the chunks; part: the planes' sums for the
// column reduction over the batch that follows (layout as in rows_bwd_resident) when fold.tagged
// is null.
// OCC: built for three workgroups per CU instead of two (80 registers, a few of them spilled; the
// addresses of the loads are computed again where the fallback loads the chunk again, which the
// build for two is better off without).  It pays when a plane has so many chunks that the two
// workgroups per CU of an XCD all belong to one plane and move in step, load - exchange - store:
// [2, 32, 128^3] fp16 (64 chunks) 147.4 -> 143.1 us; with two chunks per plane
// ([16, 64, 256, 256]) it loses, 71.0 -> 73.1 us.
template <typename T, int V, int U, bool FULL, bool OCC>
__global__ void __launch_bounds__(kPlaneThreads, OCC ? 6 : 4)
plane_bwd_single(const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ gamma,
                 const float* __restrict__ mean_in, const float* __restrict__ rstd_in, cl_word* tagged,
                 unsigned* claims, T* __restrict__ dx, float* __restrict__ part, int64_t n_rows, int n_vec, int S, int chunk_vec, int C,
                 unsigned tag, int max_polls, PlaneFold fold, unsigned* trouble) {
  __shared__ float2 sum_buf[2][16];
  __shared__ int have[kPlaneMaxChunks];
  __shared__ float inst[kWave][2];
  __shared__ float sm_s1, sm_s2;
  __shared__ int sm_fail, sm_fail_fold;
  const PlaneGeom g = plane_geom(n_rows, S);
  if (!g.active) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int64_t D = static_cast<int64_t>(n_vec) * V;
  const T* xr = x + g.row * D;
  const T* dr = dy + g.row * D;
  const int n_here = plane_chunk_vectors(g.s, S, n_vec, chunk_vec);
  const int64_t off = static_cast<int64_t>(g.s) * chunk_vec * V;
  Pack<T, V> rx[U], rd[U];
  plane_load<T, V, U, FULL, true>(xr + off, n_here, rx);
  plane_load<T, V, U, FULL, true>(dr + off, n_here, rd);
  const float mean = mean_in[g.row], rstd = rstd_in[g.row];
  const int c = static_cast<int>(g.row % C);
  const int64_t n = g.row / C;
  const float gm = gamma[c];
  if (threadIdx.x == 0) sm_fail = sm_fail_fold = 0;
  const float2 mine = plane_chunk_sums<T, V, U, FULL>(rx, rd, n_here, mean, rstd, sum_buf[0]);
  if (threadIdx.x == 0) cl_publish(tagged + (g.row * S + g.s) * 2, mine.x, mine.y, tag);
#pragma unroll
  for (int k = 0; k < U; ++k) {
    forget_derived(rx[k]);
    forget_derived(rd[k]);
  }
  if (wave == 0) {
    float pa, pb;
    if (exchange_wait_pair(tagged + (g.row * S + (lane < S ? lane : 0)) * 2, lane < S, tag, max_polls, trouble, pa, pb)) {
      const float a = group_sum<kWave>(lane < S ? pa : 0.f);
      const float b = group_sum<kWave>(lane < S ? pb : 0.f);
      if (lane == 0) {
        sm_s1 = a;
        sm_s2 = b;
      }
    } else if (lane == 0) {
      sm_fail = 1;
    }
  }
  __syncthreads();
  if (sm_fail) {
    // On its own (see the forward): dy and x are intact, dx != dy.
    const float2 t = plane_sums_alone<T, V, U, FULL>(xr, dr, mean, rstd, S, g.s, n_vec, chunk_vec, rx, rd, sum_buf,
                                                     have, tagged + g.row * S * 2, claims + g.row * S, tag);
    if (threadIdx.x == 0) {
      sm_s1 = t.x;
      sm_s2 = t.y;
    }
    plane_load<T, V, U, FULL, true, OCC>(xr + off, n_here, rx);
    plane_load<T, V, U, FULL, true, OCC>(dr + off, n_here, rd);
    __syncthreads();
  }
  const float s1 = sm_s1, s2 = sm_s2;
  if (g.s == 0 && threadIdx.x == 0) {
    if (fold.tagged == nullptr) {
      part[(n * 2 + 0) * C + c] = s2;
      part[(n * 2 + 1) * C + c] = s1;
    } else if (fold.N == 1) {
      fold.dgamma[c] = s2;
      fold.dbeta[c] = s1;
    } else {
      cl_publish(fold.tagged + g.row * 2, s2, s1, tag);
    }
  }
  // dx = rstd * gamma * (dy - s1 / D - xh * s2 / D) = ca * dy + cb * (x - mean) + cc
  const float inv_d = 1.0f / static_cast<float>(D);
  const float ca = rstd * gm;
  const float cb = -ca * s2 * inv_d * rstd;
  const float cc = -ca * s1 * inv_d;
  T* or_ = dx + g.row * D + off;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const int i = static_cast<int>(threadIdx.x) + k * kPlaneThreads;
    if (FULL || i < n_here) {
      Pack<T, V> o;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        o.v[e] = from_f32<T>(ca * to_f32(rd[k].v[e]) + (cb * (to_f32(rx[k].v[e]) - mean) + cc));
      }
      store_pack<T, V>(or_ + static_cast<int64_t>(i) * V, o);
    }
  }
  if (fold.tagged != nullptr && fold.N > 1 && g.s == 0 && n == fold.N - 1) {  // uniform in the workgroup
    const int N = fold.N;
    bool ok = false;
    float pb = 0.f, pa = 0.f;
    if (wave == 0) {
      // (patiently in any case: the planes waited for belong to workgroups started long ago)
      ok = cl_wait_pair(fold.tagged + (static_cast<int64_t>(lane < N ? lane : 0) * C + c) * 2, lane < N, tag, max_polls,
                        pb, pa);
      if (lane == 0 && !ok) sm_fail_fold = 1;
    }
    __syncthreads();
    if (sm_fail_fold) {
      // the sums of the N planes of channel c, computed here as their workgroups compute them
      for (int m = 0; m < N; ++m) {
        const int64_t row = static_cast<int64_t>(m) * C + c;
        const float2 t = plane_sums_alone<T, V, U, FULL>(x + row * D, dy + row * D, mean_in[row], rstd_in[row], S,
                                                         g.s, n_vec, chunk_vec, rx, rd, sum_buf, have,
                                                         tagged + row * S * 2, claims + row * S, tag);
        if (threadIdx.x == 0) {
          inst[m][0] = t.y;
          inst[m][1] = t.x;
        }
      }
      __syncthreads();
      if (wave == 0) {
        pb = lane < N ? inst[lane < N ? lane : 0][0] : 0.f;
        pa = lane < N ? inst[lane < N ? lane : 0][1] : 0.f;
      }
    }
    if (wave == 0) {
      const float b = group_sum<kWave>(lane < N ? pb : 0.f);
      const float a = group_sum<kWave>(lane < N ? pa : 0.f);
      if (lane == 0) {
        fold.dgamma[c] = b;
        fold.dbeta[c] = a;
      }
    }
  }
}

}  // namespace atexn
