// Channels-last InstanceNorm in ONE launch per direction, for instances that can be cut into at
// most 64 register-resident slabs: the workgroups of one instance must be on the chip together,
// on one XCD (cl_single_place below has the two grids that see to that).
//
// The two-stage kernels (cl_kernels.hip.h) read x (and dy) twice and pay a kernel boundary
// between the statistics and their use.  Here a workgroup keeps its slab in registers and the
// workgroups of an instance exchange their per-slab statistics through memory while they run:
//
//   1. every workgroup publishes the per-channel partials of its slab;
//   2. workgroup s of an instance OWNS channel s (s + S, ... when a tile has more channels than
//      the instance has slabs): one wave, a lane per slab, waits for that channel's partials,
//      folds them and publishes the channel's final statistics;
//   3. every workgroup waits for the finals of its channels (a lane per channel), derives the
//      per-channel constants and applies them to the slab it still holds.
//
// Each published value travels as an 8-byte word (value, tag) written by one store: the tag
// names this call (a process-wide call counter handed in by the host), so a word either still
// holds some older call's tag or is complete: no separate flag, no fence, no counter to clear.
// The second word of a pair carries the complemented tag, so that 64 bits of arbitrary memory
// contents would have to match before garbage in a fresh workspace is taken for data.  Readers
// use device-scope loads, which go past the vector and L2 caches' stale lines; writers use plain
// stores, which reach the L2 of their XCD: every workgroup of an instance runs on the same XCD,
// and that L2 is where those loads look.  A hop costs about 2 us, against about 3.5 us for the
// kernel boundary and the second read.
//
// Nothing here can hang: every wait is a bounded number of polls.  A workgroup whose wait runs
// out (its peers are not resident: another kernel holds the CUs; or the placement assumption
// does not hold on this device) stops relying on workgroups that may not be running: together
// with the others that have given up it computes, with the same code and therefore to the same
// bits, the partials of the slabs that are missing, from x itself, and does the duty of their
// workgroups as owners (below, at cl_look); from then on it only waits for running workgroups.
// That is why the host keeps callers that pass y == x (dx == dy) on the two-stage kernels: a
// peer may already have overwritten its part of x by then.
//
// Counterpart in the reference: the single-kernel channels-last variant that keeps an instance
// in one block's shared memory (fused_instance_norm_op.cu:1066-1165); it stops at D <= 372.
#pragma once

#include "cl_kernels.hip.h"

namespace atexn {

constexpr int kClSingleMaxCap = 64;    // channels per tile (the fallback keeps S x cap pairs in LDS)
constexpr int kClSingleMaxSlabs = 64;  // slabs per instance: one lane each in the owner's fold
constexpr int kClSingleMaxOwned = 4;   // channels one workgroup may own

// (mean, m2) of an instance from its slabs' (mean, m2), one slab per lane of a wave (lanes
// >= S hold nothing): Chan's merge of all slabs at once, as cl_fold_stats does it.
__device__ __forceinline__ void cl_fold_lanes_stats(float pm, float pq, int lane, int S, float n_full,
                                                    float n_last, float inv_d, float& mean, float& m2) {
#pragma clang fp contract(off)
  const bool in = lane < S;
  const float w = lane == S - 1 ? n_last : n_full;
  mean = group_sum<kWave>(in ? pm * w : 0.f) * inv_d;
  const float d = pm - mean;
  m2 = group_sum<kWave>(in ? pq + w * (d * d) : 0.f);
}

// Geometry of slab l of the calling workgroup's instance and channel tile (the fallback walks
// every slab with it).
__device__ __forceinline__ ClGeom cl_geom_of_slab(const ClGeom& g, int l, int64_t D, int64_t slab_len) {
  ClGeom h = g;
  h.s = l;
  h.p0 = static_cast<int64_t>(l) * slab_len;
  h.p1 = h.p0 + slab_len < D ? h.p0 + slab_len : D;
  h.slab_n = static_cast<int>(h.p1 - h.p0 < (1 << 20) ? h.p1 - h.p0 : (1 << 20));
  return h;
}

// Which (instance, slab, channel tile) the calling workgroup takes.  xm_tiles == 0: the grid is
// (N, S, channel tiles), every workgroup of the launch is on the chip at once and N is a multiple
// of the XCD count, which puts an instance's workgroups on one XCD.  xm_tiles > 0 (the number of
// channel tiles): a one-dimensional, XCD-major grid for any N and any number of workgroups:
// workgroups are dealt to the 8 XCDs in turn and each XCD starts its workgroups in index order, so
// workgroup b takes slab (b / 8) % S of unit ((b / 8) / S) * 8 + b % 8, a unit being an (instance,
// channel tile) pair: the S workgroups of a unit are consecutive workgroups of one XCD, resident
// together when S is at most what an XCD holds, and wait only for each other.  False: the
// workgroup has nothing to do (the grid is padded to whole units per XCD).
constexpr int kClSingleXcds = 8;
__device__ __forceinline__ bool cl_single_place(int64_t N, int S, int xm_tiles, int64_t& n, int& s, int& ct) {
  if (xm_tiles == 0) {
    n = blockIdx.x;
    s = static_cast<int>(blockIdx.y);
    ct = static_cast<int>(blockIdx.z);
    return true;
  }
  const unsigned b = blockIdx.x;
  const unsigned xcd = b % kClSingleXcds, j = b / kClSingleXcds;
  const int64_t unit = static_cast<int64_t>(j / static_cast<unsigned>(S)) * kClSingleXcds + xcd;
  s = static_cast<int>(j % static_cast<unsigned>(S));
  n = unit / xm_tiles;
  ct = static_cast<int>(unit % xm_tiles);
  return unit < N * xm_tiles;
}

// A workgroup's fallback (a wait of its has run out) starts with a look: which slabs of instance n
// have published the partials of all the channels of this tile (have[l] = 1)?  One look per
// (slab, channel), 256 at a time.  The missing slabs then get computed, each once, by the
// workgroups that have given up: round by round a workgroup looks, claims ONE missing slab that
// nobody has claimed yet (cl_claim_missing: a compare-and-swap of the call's tag into the slab's
// claim word), computes its partials as the slab's own workgroup would, publishes them and looks
// again; when nothing is left to claim, whatever is still missing is in the hands of a running
// workgroup and only has to be waited for.  (When the workgroups of an instance cannot be
// resident together because another kernel fills part of the chip, the resident ones thus share
// out the slabs of the absent ones instead of each redoing the whole instance; the absent ones,
// once started, find everything published, publish their own again with the same bits and go on.)
// Whoever publishes a slab's partials also does its workgroup's duty as an owner (step 2 above)
// for the channels that the slab owns, so every channel's finals come from a running workgroup.
// Contains barriers; have is valid for every thread afterwards.
__device__ __forceinline__ void cl_look(const cl_word* tagged, int64_t n, int S, int C, int c_base, int cap_here,
                                        unsigned tag, int (&have)[kClSingleMaxSlabs]) {
  __syncthreads();  // whatever read have before is done
  if (threadIdx.x < kClSingleMaxSlabs) have[threadIdx.x] = 1;
  __syncthreads();
  const int lc = threadIdx.x & (kClSingleMaxCap - 1);
  for (int l = threadIdx.x / kClSingleMaxCap; l < S; l += kClThreads / kClSingleMaxCap) {
    if (lc < cap_here) {
      const cl_word* pair = tagged + ((n * S + l) * C + c_base + lc) * 2;
      const cl_word w0 = cl_peek(pair);
      const cl_word w1 = cl_peek(pair + 1);
      if (static_cast<unsigned>(w0 >> 32) != tag || static_cast<unsigned>(w1 >> 32) != ~tag) have[l] = 0;
    }
  }
  __syncthreads();
}
// One round of that: -1 when no missing slab is left to claim, else the slab this workgroup is to
// compute.  claims: the claim words of the instance's slabs for this tile.  Contains barriers.
__device__ __forceinline__ int cl_claim_missing(unsigned* claims, int S, int s_self, unsigned tag,
                                                const int (&have)[kClSingleMaxSlabs]) {
  __shared__ int sm_pick;
  if (threadIdx.x < kWave) {
    // a lane per slab looks at its claim word; the candidates are then tried in turn, starting
    // behind the workgroup's own slab (so that the workgroups spread over the missing ones)
    const int lane = threadIdx.x;
    const int l = (s_self + 1 + lane) % S;  // lane i: the i-th slab behind this one (i < S)
    bool open_ = false;
    if (lane < S && !have[l]) {
      open_ = __hip_atomic_load(claims + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != tag;
    }
    unsigned long long cand = __ballot(open_);
    int pick = -1;
    while (cand != 0 && pick < 0) {  // uniform over the wave
      const int first = __builtin_ctzll(cand);
      int got = 0;
      if (lane == first) {
        unsigned cur = __hip_atomic_load(claims + l, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        got = cur != tag && __hip_atomic_compare_exchange_strong(claims + l, &cur, tag, __ATOMIC_RELAXED,
                                                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                  ? 1 : 0;
      }
      got = __shfl(got, first, kWave);
      if (got) pick = (s_self + 1 + first) % S;
      cand &= cand - 1;
    }
    if (lane == 0) sm_pick = pick;
  }
  __syncthreads();
  return sm_pick;
}
// The first slab whose partials have not been seen (-1: none); the same in every thread.
__device__ __forceinline__ int cl_first_missing(int S, const int (&have)[kClSingleMaxSlabs]) {
  for (int l = 0; l < S; ++l) {
    if (!have[l]) return l;
  }
  return -1;
}
// Polls that a workgroup allows for values that it has published itself, has just seen, or knows
// to be in the hands of a running workgroup to show up in its device-scope loads: they are on
// their way, this only bounds the wait.
constexpr int kClOwnPolls = 1 << 16;
// The wait for such values.  Should they not show up after all, the result is marked (NaN) rather
// than computed from whatever the words held.
__device__ __forceinline__ void cl_wait_own(const cl_word* pair, bool want, unsigned tag, float& a, float& b) {
  if (!cl_wait_pair(pair, want, tag, kClOwnPolls, a, b)) a = b = __builtin_nanf("");
}

// Channel tiles of the launch, on either grid.
__device__ __forceinline__ int gridDim_tiles(int xm_tiles) {
  return xm_tiles == 0 ? static_cast<int>(gridDim.z) : xm_tiles;
}

// Whether the waits of a kernel adapt to a shared GPU (exchange_wait_pair).  The kernels of small
// slabs (four vectors per thread) do not: their launches are a few microseconds long, of which
// the adaptive wait's code - never its read of the record - cost 0.4 of 14 in a forward + backward
// step ([8, 64^2, 64], [2, 16^3, 128], [4, 64^2, 32] fp16), and the 300 polls that a wait on a
// shared GPU then runs to are bounded by the same few workgroups.  With eight vectors per thread
// the cost is within the noise (config 3: 20.35 against 20.5 us).
template <int U>
__device__ __forceinline__ constexpr bool cl_single_adapts() {
  return U >= 8;
}

// ------------------------------------------------------------------------------ forward
// tagged: [N][S][C] pairs (mean, m2) of the slabs; finals: [N][C] pairs (mean, inverse std);
// claims: [N][tiles][S] claim words.
// Grid: see cl_single_place; tile of at most 64 channels.
// OCC: compiled for four workgroups per CU instead of two (128 VGPRs, a few values in scratch
// memory): an XCD then has the workgroups of two instances in flight, one loading while the
// other waits for its exchange.  Pays on the XCD-major grid with more instances than the chip
// holds at once ([16, 128^2, 64] fp16 forward 18.3 -> 14.7 us, [64, 128^2, 64] 68.1 -> 59.3 us);
// a launch that fits the chip anyway loses a little (config 3: 9.97 -> 10.4 us) and keeps OCC off.
template <typename T, int V, int U, bool FULL, bool OCC>
__global__ void __launch_bounds__(kClThreads, OCC ? 4 : 2)
cl_fwd_single(const T* __restrict__ x, cl_word* tagged, cl_word* finals, unsigned* claims,
              const float* __restrict__ gamma,
              const float* __restrict__ beta, T* __restrict__ y, float* __restrict__ mean_out,
              float* __restrict__ rstd_out, int64_t N, int64_t D, int C, int S, int tpp_shift, int64_t slab_len,
              float eps, unsigned tag, int max_polls, int xm_tiles, unsigned* trouble) {
  __shared__ float lds[V * kClThreads];
  __shared__ int have[kClSingleMaxSlabs];
  __shared__ int mine[kClSingleMaxSlabs];
  __shared__ float sm_mean[kClSingleMaxCap], sm_sc[kClSingleMaxCap], sm_bt[kClSingleMaxCap];
  __shared__ int sm_fail;
  const int CV = C / V;
  const int TPP = 1 << tpp_shift;
  const int cap = TPP * V;
  int64_t n_;
  int s_, ct_;
  if (!cl_single_place(N, S, xm_tiles, n_, s_, ct_)) return;
  const ClGeom g = cl_geom_at<false>(n_, s_, ct_, tpp_shift, CV, C, V, D, slab_len);
  const int c_base = g.ct * cap;
  const int cap_here = C - c_base < cap ? C - c_base : cap;
  const int lane = threadIdx.x & (kWave - 1);
  unsigned* const record = cl_single_adapts<U>() ? trouble : nullptr;
  const int wave = threadIdx.x / kWave;
  const float inv_d = 1.0f / static_cast<float>(D);
  const float n_full = static_cast<float>(slab_len);
  const float n_last = static_cast<float>(D - static_cast<int64_t>(S - 1) * slab_len);
  if (threadIdx.x == 0) sm_fail = 0;
  Pack<T, V> raw[U];
  bool ok[U];
  cl_load_slab<T, V, U, false, FULL>(x + (g.n * D + g.p0) * C, g, C, raw, ok);
  // what the gathering lanes of wave 0 need besides the finals
  float gmc = 0.f, btc = 0.f;
  if (wave == 0 && lane < cap_here) {
    gmc = gamma[c_base + lane];
    btc = beta[c_base + lane];
  }
  float mean[V], m2[V];
  cl_resident_stats<T, V, U>(raw, ok, 1.0f / static_cast<float>(g.p1 - g.p0), TPP, lds, mean, m2);
  if (g.ch_ok && g.slot == 0) {
    cl_word* o = tagged + ((g.n * S + g.s) * C + g.coff) * 2;
#pragma unroll
    for (int i = 0; i < V; ++i) cl_publish(o + 2 * i, mean[i], m2[i], tag);
  }
  if (wave == 0) {
    bool fail = false;
    // the channels this workgroup owns: a lane per slab
    for (int lc = g.s; lc < cap_here; lc += S) {
      const int c = c_base + lc;
      float pm, pq;
      if (!exchange_wait_pair(tagged + ((g.n * S + (lane < S ? lane : 0)) * C + c) * 2, lane < S, tag, max_polls, record, pm, pq)) {
        fail = true;
        break;
      }
      float mu, q;
      cl_fold_lanes_stats(pm, pq, lane, S, n_full, n_last, inv_d, mu, q);
      if (lane == 0) {
        const float rs = rsqrtf(__builtin_fmaf(q, inv_d, eps));
        cl_publish(finals + (g.n * C + c) * 2, mu, rs, tag);
        mean_out[g.n * C + c] = mu;
        rstd_out[g.n * C + c] = rs;
      }
    }
    // the finals of this tile's channels: a lane per channel
    if (!fail) {
      float fm, frs;
      const bool want = lane < cap_here;
      if (exchange_wait_pair(finals + (g.n * C + c_base + (want ? lane : 0)) * 2, want, tag, max_polls, record, fm, frs)) {
        if (want) {
          sm_mean[lane] = fm;
          sm_sc[lane] = gmc * frs;
          sm_bt[lane] = btc;
        }
      } else {
        fail = true;
      }
    }
    if (fail && lane == 0) sm_fail = 1;
  }
  __syncthreads();
  if (sm_fail) {
    // The partials of every slab of the instance that have not arrived get computed as their
    // workgroups compute them and published like theirs, each by one of the workgroups that have
    // given up.  Whoever publishes a slab's partials also does its workgroup's duty as an owner:
    // it folds the channels that the slab owns and publishes their finals (the absent workgroup,
    // once it runs, does both again, to the same bits).  So every channel's finals come from a
    // running workgroup, and all that is left is to wait for them.  The slabs pass through the
    // registers of the workgroup's own slab, which is loaded again at the end (x is intact:
    // y != x).
    unsigned* my_claims = claims + (g.n * gridDim_tiles(xm_tiles) + g.ct) * S;
    int n_mine = 0;  // uniform
    for (int round = 0; round < S; ++round) {
      cl_look(tagged, g.n, S, C, c_base, cap_here, tag, have);
      const int l = cl_claim_missing(my_claims, S, g.s, tag, have);
      if (l < 0) break;  // uniform
      if (threadIdx.x == 0) mine[n_mine] = l;
      ++n_mine;
      const ClGeom h = cl_geom_of_slab(g, l, D, slab_len);
      cl_load_slab<T, V, U, false, FULL>(x + (h.n * D + h.p0) * C, h, C, raw, ok);
      float mm[V], qq[V];
      cl_resident_stats<T, V, U>(raw, ok, 1.0f / static_cast<float>(h.p1 - h.p0), TPP, lds, mm, qq);
      if (g.ch_ok && g.slot == 0) {
        cl_word* o = tagged + ((g.n * S + l) * C + g.coff) * 2;
#pragma unroll
        for (int i = 0; i < V; ++i) cl_publish(o + 2 * i, mm[i], qq[i], tag);
      }
    }
    __syncthreads();  // mine is written
    for (int k = -1; k < n_mine; ++k) {
      const int sk = k < 0 ? g.s : mine[k];
      for (int lc = sk + wave * S; lc < cap_here; lc += (kClThreads / kWave) * S) {
        const int c = c_base + lc;
        float pm, pq;
        cl_wait_own(tagged + ((g.n * S + (lane < S ? lane : 0)) * C + c) * 2, lane < S, tag, pm, pq);
        float mu, q;
        cl_fold_lanes_stats(pm, pq, lane, S, n_full, n_last, inv_d, mu, q);
        if (lane == 0) {
          const float rs = rsqrtf(__builtin_fmaf(q, inv_d, eps));
          cl_publish(finals + (g.n * C + c) * 2, mu, rs, tag);
          mean_out[g.n * C + c] = mu;
          rstd_out[g.n * C + c] = rs;
        }
      }
    }
    if (wave == 0) {
      float fm, frs;
      const bool want = lane < cap_here;
      cl_wait_own(finals + (g.n * C + c_base + (want ? lane : 0)) * 2, want, tag, fm, frs);
      if (want) {
        sm_mean[lane] = fm;
        sm_sc[lane] = gmc * frs;
        sm_bt[lane] = btc;
      }
    }
    cl_load_slab<T, V, U, false, FULL>(x + (g.n * D + g.p0) * C, cl_geom_again(g), C, raw, ok);
    __syncthreads();
  }
  if (g.ch_ok) {
    ClFwdCoef<V, false> k;
    k.load(g, tpp_shift, sm_mean, sm_sc, sm_bt);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) {
        store_pack<T, V>(y + (g.n * D + g.p0) * C + cl_slab_offset(g, C, u), k.template apply<T>(raw[u]));
      }
    }
  }
}

// ----------------------------------------------------------------------------- backward
// tagged: [N][S][C] pairs (sum dy * xh, sum dy) of the slabs; finals: [N][C] pairs of the
// instances' sums, for the workgroups of the instance; finals_dev: the same pairs written
// through to memory, for the workgroups of instance 0, which own the fold over the instances:
// the owner of channel c there adds up the N pairs of c (a lane per instance) into dgamma[c]
// and dbeta[c] after it has stored its dx.  N <= 64.  finals_dev == nullptr (the XCD-major grid,
// whose workgroups are not all on the chip together): the owners leave the instances' sums at
// o0[n * o_stride + c] (sum dy * xh) and o1[n * o_stride + c] (sum dy) instead: dgamma / dbeta
// themselves for a single instance, partial rows for a col_reduce launch otherwise.
// OCC: built for four workgroups per CU (128 registers, a dozen of the 16-bit kernel's 138 in
// scratch memory), so that an XCD holds two instances of 64 slabs at a time; the plain build
// already runs three per CU.
template <typename T, int V, int U, bool FULL, bool OCC>
__global__ void __launch_bounds__(kClThreads, OCC ? 4 : 2)
cl_bwd_single(const T* __restrict__ dy, const T* __restrict__ x, const float* __restrict__ gamma,
              const float* __restrict__ mean_in, const float* __restrict__ rstd_in, cl_word* tagged,
              cl_word* finals, cl_word* finals_dev, unsigned* claims, T* __restrict__ dx, float* __restrict__ dgamma,
              float* __restrict__ dbeta, int N, int64_t D, int C, int S, int tpp_shift, int64_t slab_len,
              unsigned tag, int max_polls, int xm_tiles, float* __restrict__ o0, float* __restrict__ o1,
              int64_t o_stride, unsigned* trouble) {
  __shared__ float lds[2 * V * kClThreads];
  __shared__ int have[kClSingleMaxSlabs];
  __shared__ int mine[kClSingleMaxSlabs];
  __shared__ float sm_mu[kClSingleMaxCap], sm_sc[kClSingleMaxCap], sm_ca[kClSingleMaxCap], sm_cb[kClSingleMaxCap];
  __shared__ float inst[kClSingleMaxOwned][kWave][2];
  __shared__ int sm_fail, sm_fail_dev;
  const int CV = C / V;
  const int TPP = 1 << tpp_shift;
  const int cap = TPP * V;
  int64_t n_;
  int s_, ct_;
  if (!cl_single_place(N, S, xm_tiles, n_, s_, ct_)) return;
  const ClGeom g = cl_geom_at<false>(n_, s_, ct_, tpp_shift, CV, C, V, D, slab_len);
  const int c_base = g.ct * cap;
  const int cap_here = C - c_base < cap ? C - c_base : cap;
  const int lane = threadIdx.x & (kWave - 1);
  unsigned* const record = cl_single_adapts<U>() ? trouble : nullptr;
  const int wave = threadIdx.x / kWave;
  const float inv_d = 1.0f / static_cast<float>(D);
  if (threadIdx.x == 0) sm_fail = sm_fail_dev = 0;
  Pack<T, V> rx[U], rd[U];
  bool ok[U];
  cl_load_slab<T, V, U, true, FULL>(x + (g.n * D + g.p0) * C, g, C, rx, ok);
  cl_load_slab<T, V, U, true, FULL>(dy + (g.n * D + g.p0) * C, g, C, rd, ok);
  float mu[V], rs[V];
#pragma unroll
  for (int i = 0; i < V; ++i) mu[i] = rs[i] = 0.f;
  if (g.ch_ok) {
    load_f32<V>(mean_in + g.n * C + g.coff, mu);
    load_f32<V>(rstd_in + g.n * C + g.coff, rs);
  }
  // what the gathering lanes of wave 0 need besides the finals
  float gmc = 0.f, muc = 0.f, rsc = 0.f;
  if (wave == 0 && lane < cap_here) {
    gmc = gamma[c_base + lane];
    muc = mean_in[g.n * C + c_base + lane];
    rsc = rstd_in[g.n * C + c_base + lane];
  }
  float acc[2 * V];
  cl_resident_sums<T, V, U>(rx, rd, ok, mu, rs, TPP, lds, acc);
  if (g.ch_ok && g.slot == 0) {
    cl_word* o = tagged + ((g.n * S + g.s) * C + g.coff) * 2;
#pragma unroll
    for (int i = 0; i < V; ++i) cl_publish(o + 2 * i, acc[i], acc[V + i], tag);
  }
  // constants of dx = sc * dy + (ca * (x - mu) + cb) from an instance's sums (b = sum dy * xh,
  // a = sum dy), as cl_fold_sums derives them
  auto constants = [&](int lc, float gm, float m, float r, float b, float a) {
#pragma clang fp contract(off)
    const float sc = gm * r;
    sm_mu[lc] = m;
    sm_sc[lc] = sc;
    sm_ca[lc] = -(sc * r) * (b * inv_d);
    sm_cb[lc] = -sc * (a * inv_d);
  };
  if (wave == 0) {
    bool fail = false;
    for (int lc = g.s; lc < cap_here; lc += S) {
      const int c = c_base + lc;
      float pb, pa;
      if (!exchange_wait_pair(tagged + ((g.n * S + (lane < S ? lane : 0)) * C + c) * 2, lane < S, tag, max_polls, record, pb, pa)) {
        fail = true;
        break;
      }
      const float b = group_sum<kWave>(lane < S ? pb : 0.f);
      const float a = group_sum<kWave>(lane < S ? pa : 0.f);
      if (lane == 0) {
        cl_publish(finals + (g.n * C + c) * 2, b, a, tag);
        if (finals_dev != nullptr) {
          cl_publish_device(finals_dev + (g.n * C + c) * 2, b, a, tag);
        } else {
          o0[g.n * o_stride + c] = b;
          o1[g.n * o_stride + c] = a;
        }
      }
    }
    if (!fail) {
      float fb_, fa_;
      const bool want = lane < cap_here;
      if (exchange_wait_pair(finals + (g.n * C + c_base + (want ? lane : 0)) * 2, want, tag, max_polls, record, fb_, fa_)) {
        if (want) constants(lane, gmc, muc, rsc, fb_, fa_);
      } else {
        fail = true;
      }
    }
    if (fail && lane == 0) sm_fail = 1;
  }
  __syncthreads();
  // The sums of channel c of instance n2 from its slabs' sums (all of them are there or on their
  // way after ensure_instance): a lane per slab, the whole wave must call.
  auto fold_slabs = [&](int64_t n2, int c, float& b, float& a) {
    float pb, pa;
    cl_wait_own(tagged + ((n2 * S + (lane < S ? lane : 0)) * C + c) * 2, lane < S, tag, pb, pa);
    b = group_sum<kWave>(lane < S ? pb : 0.f);
    a = group_sum<kWave>(lane < S ? pa : 0.f);
  };
  // The owner's duty for slab sk of instance n2: the sums of the channels that the slab owns,
  // published for the instance's workgroups and for the fold over the batch.
  auto owner_duty = [&](int64_t n2, int sk) {
    for (int lc = sk + wave * S; lc < cap_here; lc += (kClThreads / kWave) * S) {
      const int c = c_base + lc;
      float b, a;
      fold_slabs(n2, c, b, a);
      if (lane == 0) {
        cl_publish(finals + (n2 * C + c) * 2, b, a, tag);
        if (finals_dev != nullptr) {
          cl_publish_device(finals_dev + (n2 * C + c) * 2, b, a, tag);
        } else {
          o0[n2 * o_stride + c] = b;
          o1[n2 * o_stride + c] = a;
        }
      }
    }
  };
  // On its own, for instance n2 and this workgroup's tile: the sums of every slab that have not
  // arrived, computed as their workgroups compute them and published like theirs.  The slabs pass
  // through the registers of the workgroup's own slab (x and dy are intact: dx aliases neither),
  // which the caller loads again if it still needs it.
  int n_mine = 0;  // slabs of the instance that ensure_instance computed here (uniform); they are in mine[]
  auto ensure_instance = [&](int64_t n2) {
    float mu2[V], rs2[V];
#pragma unroll
    for (int i = 0; i < V; ++i) mu2[i] = rs2[i] = 0.f;
    if (g.ch_ok) {
      load_f32<V>(mean_in + n2 * C + g.coff, mu2);
      load_f32<V>(rstd_in + n2 * C + g.coff, rs2);
    }
    unsigned* my_claims = claims + (n2 * gridDim_tiles(xm_tiles) + g.ct) * S;
    // Another instance's workgroups sit on another XCD: what they publish with plain stores is
    // not to be seen from here before their L2 lets go of it, and what is published from here
    // they do not see either.  So for another instance (the fold over the batch, below) nothing
    // is claimed and no claim is honoured: whatever this workgroup cannot see it computes itself,
    // for its own use.
    const bool same_xcd = n2 == g.n;
    n_mine = 0;
    for (int round = 0; round < S; ++round) {
      cl_look(tagged, n2, S, C, c_base, cap_here, tag, have);
      const int l = same_xcd ? cl_claim_missing(my_claims, S, g.s, tag, have) : cl_first_missing(S, have);
      if (l < 0) break;  // uniform
      if (same_xcd) {
        if (threadIdx.x == 0) mine[n_mine] = l;
        ++n_mine;
      }
      const ClGeom h = cl_geom_of_slab(g, l, D, slab_len);
      cl_load_slab<T, V, U, true, FULL>(x + (n2 * D + h.p0) * C, h, C, rx, ok);
      cl_load_slab<T, V, U, true, FULL>(dy + (n2 * D + h.p0) * C, h, C, rd, ok);
      float a2[2 * V];
      cl_resident_sums<T, V, U>(rx, rd, ok, mu2, rs2, TPP, lds, a2);
      if (g.ch_ok && g.slot == 0) {
        cl_word* o = tagged + ((n2 * S + l) * C + g.coff) * 2;
#pragma unroll
        for (int i = 0; i < V; ++i) cl_publish(o + 2 * i, a2[i], a2[V + i], tag);
      }
    }
    __syncthreads();  // mine is written
    // whoever publishes a slab's sums also does its workgroup's duty as an owner (the absent
    // workgroup, once it runs, does both again, to the same bits): every channel's sums thus
    // come from a running workgroup
    for (int k = 0; k < n_mine; ++k) owner_duty(n2, mine[k]);
  };
  if (sm_fail) {
    // What is missing of the instance's sums, this workgroup's own duty as an owner (again, if
    // the wait that ran out was the one for the sums of the instance), and then all that is left
    // is to wait for every channel's sums: they come from running workgroups.
    ensure_instance(g.n);
    owner_duty(g.n, g.s);
    if (wave == 0) {
      float fb_, fa_;
      const bool want = lane < cap_here;
      cl_wait_own(finals + (g.n * C + c_base + (want ? lane : 0)) * 2, want, tag, fb_, fa_);
      if (want) constants(lane, gmc, muc, rsc, fb_, fa_);
    }
    const ClGeom g2 = cl_geom_again(g);
    cl_load_slab<T, V, U, true, FULL>(x + (g.n * D + g.p0) * C, g2, C, rx, ok);
    cl_load_slab<T, V, U, true, FULL>(dy + (g.n * D + g.p0) * C, g2, C, rd, ok);
    __syncthreads();
  }
  // The owners of instance 0 also fold the instances' sums into dgamma / dbeta (below, after
  // their dx is on its way).  The other instances' owners published their sums a hop ago: a first
  // look now, whose round trip passes under the stores, usually finds them.
  const bool folds_instances = finals_dev != nullptr && g.n == 0 && g.s < cap_here;  // uniform over the workgroup
  float eb = 0.f, ea = 0.f;
  bool early = false;
  if (folds_instances && wave == 0 && max_polls > 0) {
    early = cl_try_pair(finals_dev + (static_cast<int64_t>(lane < N ? lane : 0) * C + c_base + g.s) * 2, lane < N, tag,
                        eb, ea);
  }
  if (g.ch_ok) {
    ClBwdCoef<V, false> k;
    k.load(g, tpp_shift, sm_mu, sm_sc, sm_ca, sm_cb);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (ok[u]) {
        store_pack<T, V>(dx + (g.n * D + g.p0) * C + cl_slab_offset(g, C, u),
                         k.template apply<T>(rx[u], rd[u]));
      }
    }
  }
  // dgamma / dbeta: the owners of instance 0 add up the instances' sums, a lane per instance
  // (the first owned channel's may have arrived with the early look)
  if (!folds_instances) return;
  if (wave == 0) {
    bool fail = false;
    for (int lc = g.s; lc < cap_here; lc += S) {
      const int c = c_base + lc;
      float pb = eb, pa = ea;
      if (!(early && lc == g.s) &&
          // (patiently in any case: the other instances do not depend on this workgroup)
          !cl_wait_pair(finals_dev + (static_cast<int64_t>(lane < N ? lane : 0) * C + c) * 2, lane < N, tag,
                        max_polls, pb, pa)) {
        fail = true;
        break;
      }
      const float b = group_sum<kWave>(lane < N ? pb : 0.f);
      const float a = group_sum<kWave>(lane < N ? pa : 0.f);
      if (lane == 0) {
        dgamma[c] = b;
        dbeta[c] = a;
      }
    }
    if (fail && lane == 0) sm_fail_dev = 1;
  }
  __syncthreads();
  if (sm_fail_dev) {
    // every instance's sums for the owned channels, from its slabs' sums (what has not arrived
    // of those is computed here)
    for (int n2 = 0; n2 < N; ++n2) {
      ensure_instance(n2);
      int k = 0;
      for (int lc = g.s; lc < cap_here; lc += S, ++k) {
        if (wave == 0) {
          float b, a;
          fold_slabs(n2, c_base + lc, b, a);
          if (lane == 0) {
            inst[k][n2][0] = b;
            inst[k][n2][1] = a;
          }
        }
      }
    }
    __syncthreads();
    if (wave == 0) {
      int k = 0;
      for (int lc = g.s; lc < cap_here; lc += S, ++k) {
        const float b = group_sum<kWave>(lane < N ? inst[k][lane][0] : 0.f);
        const float a = group_sum<kWave>(lane < N ? inst[k][lane][1] : 0.f);
        if (lane == 0) {
          dgamma[c_base + lc] = b;
          dbeta[c_base + lc] = a;
        }
      }
    }
  }
}

}  // namespace atexn
