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
// on the vector paths and sizeof(T) on the element-wise paths).  The type is only
// element-aligned: gfx950 global accesses of 16 bytes work at any element alignment (measured
// at 97 % of the aligned copy rate), so rows may start anywhere.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
typedef unsigned int u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
// 16 bytes as one register quad, aligned like the element type it stands for
template <size_t ELEM_BYTES>
struct Bits16 {
  using type = u32x4_a4;
};
template <>
struct Bits16<2> {
  using type = u32x4_a2;
};

template <typename T, int V>
struct Pack {
  T v[V];
};
struct F32x4 {
  float v[4];
};

// (16 bytes are loaded as ONE vector value and then viewed as elements: loaded as a struct of
// elements, the optimiser may cut the access into per-element pieces when the value travels
// through a loop-carried copy, and reassemble them into 2- and 4-byte loads.)
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack(const T* p) {
  if constexpr (sizeof(T) * V == 16) {
    using u32x4_u = typename Bits16<sizeof(T)>::type;
    const u32x4 bits = *reinterpret_cast<const u32x4_u*>(p);
    Pack<T, V> r;
    __builtin_memcpy(&r, &bits, 16);
    return r;
  } else {
    return *reinterpret_cast<const Pack<T, V>*>(p);
  }
}
// The last read of an input: by the second stage of a two-stage kernel, where the non-temporal
// hint keeps these lines from displacing what is still to be read (measured: 0-3 % off the
// backward of the 268 MB cases, 9 % off [10, 10^7]), and by every single-pass backward kernel,
// which reads x and dy once and last: fp16 backward alone [262144, 128] 39.5 -> 36.5 us,
// [16384, 4096] 77.7 -> 71.6 us; forward + backward in a row [8192, 1024] 20.9 -> 18.5 us,
// [2048, 12288] 57.6 -> 54.7 us, [8, 64, 128, 128] channel-first 15.5 -> 14.7 us.  (The forward
// kernels keep plain loads: the backward reads the same x afterwards.)
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack_last(const T* p) {
  if constexpr (sizeof(T) * V == 16) {
    using u32x4_u = typename Bits16<sizeof(T)>::type;
    const u32x4 bits = __builtin_nontemporal_load(reinterpret_cast<const u32x4_u*>(p));
    Pack<T, V> r;
    __builtin_memcpy(&r, &bits, 16);
    return r;
  } else {
    return load_pack<T, V>(p);
  }
}
// Output tensors (y, dx) are written once and never read back by these kernels, so their
// stores carry the non-temporal hint: the lines do not compete with the inputs for L2 and
// drain as a stream.  Measured on MI355X against plain stores: forward 8.7 -> 6.3 us at
// [8192, 1024] fp16, 157 -> 128 us at 268 MB per tensor.
template <typename T, int V>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, V>& v) {
  constexpr int kBytes = static_cast<int>(sizeof(T)) * V;
  if constexpr (kBytes == 16) {
    using u32x4_u = typename Bits16<sizeof(T)>::type;
    u32x4 bits;
    __builtin_memcpy(&bits, &v, 16);
    __builtin_nontemporal_store(bits, reinterpret_cast<u32x4_u*>(p));
  } else if constexpr (kBytes == 4) {
    unsigned int bits;
    __builtin_memcpy(&bits, &v, 4);
    __builtin_nontemporal_store(bits, reinterpret_cast<unsigned int*>(p));
  } else if constexpr (kBytes == 2) {
    unsigned short bits;
    __builtin_memcpy(&bits, &v, 2);
    __builtin_nontemporal_store(bits, reinterpret_cast<unsigned short*>(p));
  } else {
    *reinterpret_cast<Pack<T, V>*>(p) = v;
  }
}

// Makes the compiler forget what it knows about a register-resident vector: values derived
// from it before this point (its float conversions) cannot be kept alive in its place, so only
// the raw 16 bytes stay in registers across a long wait.
template <typename T, int V>
__device__ __forceinline__ void forget_derived(Pack<T, V>& v) {
  if constexpr (sizeof(T) * V == 16) {
    u32x4 bits;
    __builtin_memcpy(&bits, &v, 16);
    asm volatile("" : "+v"(bits));
    __builtin_memcpy(&v, &bits, 16);
  }
}

// Between the loads of a batch (up to two arrays of N <= 4 vectors, or one of N <= 8) and their
// first use: one empty asm statement takes every vector of the batch as an operand, so the
// compiler must have issued all the loads before it and cannot sink a load down to its use
// (left alone it sometimes emits load, wait, use, load, wait, use, ... and a batch then pays
// one memory latency per load instead of one per batch).
// Makes the compiler wait, at this point, for the loads that a[0..N) come from (an empty asm
// statement per value, which takes it as an operand).  Before a loop that prefetches: a wait
// left to the first use inside the loop is counted in operations still allowed in flight as
// seen from the loop's entry, and on the way round the loop it then holds up for the prefetch
// that was just issued.
template <int N>
__device__ __forceinline__ void values_arrived(float (&a)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) asm volatile("" : "+v"(a[i]));
}

template <typename T, int V, int N>
__device__ __forceinline__ void batch_loaded(Pack<T, V> (&a)[N]) {
  static_assert(N <= 8, "at most 8 vectors per statement");
  if constexpr (sizeof(T) * V == 16) {
    u32x4 b[8];
#pragma unroll
    for (int i = 0; i < N; ++i) __builtin_memcpy(&b[i], &a[i], 16);
#pragma unroll
    for (int i = N; i < 8; ++i) b[i] = b[0];
    if constexpr (N <= 1) asm volatile("" : "+v"(b[0]));
    else if constexpr (N <= 2) asm volatile("" : "+v"(b[0]), "+v"(b[1]));
    else if constexpr (N <= 4) asm volatile("" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
    else asm volatile("" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7]));
#pragma unroll
    for (int i = 0; i < N; ++i) __builtin_memcpy(&a[i], &b[i], 16);
  }
}
template <typename T, int V, int N>
__device__ __forceinline__ void batch_loaded(Pack<T, V> (&a)[N], Pack<T, V> (&c)[N]) {
  static_assert(N <= 4, "at most 8 vectors per statement");
  if constexpr (sizeof(T) * V == 16) {
    u32x4 b[8];
#pragma unroll
    for (int i = 0; i < N; ++i) {
      __builtin_memcpy(&b[i], &a[i], 16);
      __builtin_memcpy(&b[4 + i], &c[i], 16);
    }
#pragma unroll
    for (int i = N; i < 4; ++i) {
      b[i] = b[0];
      b[4 + i] = b[4];
    }
    if constexpr (N <= 2) asm volatile("" : "+v"(b[0]), "+v"(b[1]), "+v"(b[4]), "+v"(b[5]));
    else asm volatile("" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7]));
#pragma unroll
    for (int i = 0; i < N; ++i) {
      __builtin_memcpy(&a[i], &b[i], 16);
      __builtin_memcpy(&c[i], &b[4 + i], 16);
    }
  }
}

// The first cnt (0 <= cnt <= V) elements of a vector; the rest read as zero / are not written.
// cnt == V takes the single wide access.
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack_n(const T* p, int cnt) {
  if (cnt == V) return load_pack<T, V>(p);
  Pack<T, V> r;
#pragma unroll
  for (int i = 0; i < V; ++i) r.v[i] = i < cnt ? p[i] : T(0);
  return r;
}
template <typename T, int V>
__device__ __forceinline__ void store_pack_n(T* p, const Pack<T, V>& v, int cnt) {
  if (cnt == V) {
    store_pack<T, V>(p, v);
    return;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (i < cnt) p[i] = v.v[i];
  }
}

// Elements lo .. V-1 of a vector (lo == 0: the single wide access).  The partial case is a
// plain predicated element loop: a switch over lo with chunked stores measured slower.
template <typename T, int V>
__device__ __forceinline__ void store_pack_from(T* p, const Pack<T, V>& v, int lo) {
  if (lo == 0) {
    store_pack<T, V>(p, v);
    return;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (i >= lo) p[i] = v.v[i];
  }
}

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);  // round-to-nearest-even for f16 / bf16
}

// Half storage: the conversion to float can ride on the multiply-add that consumes the value
// (v_fma_mix_f32 takes a half operand as it is), which saves the separate v_cvt_f32_f16 per
// element.  The compiler only forms it from an fma, and folds fma(x, 1, c) back into an add, so
// the plain sums and differences below multiply by a 1.0f it cannot see through (mix_one()).
// x * 1 is exact, so each result has the bits of the converted-then-added form.  Kernels whose
// arithmetic trails their loads (a register-resident slab: every load is issued, then every
// element is touched twice) are bound by these instruction counts, not by memory.
__device__ __forceinline__ float mix_one() {
  float one = 1.0f;
  asm volatile("" : "+v"(one));
  return one;
}
template <typename T>
__device__ __forceinline__ float add_f32(float acc, T x, float one) {  // acc + float(x)
  if constexpr (sizeof(T) == 2 && !__is_same(T, bf16_t)) return __builtin_fmaf(static_cast<float>(x), one, acc);
  else return acc + to_f32(x);
}
template <typename T>
__device__ __forceinline__ float sub_f32(T x, float m, float one) {  // float(x) - m
  if constexpr (sizeof(T) == 2 && !__is_same(T, bf16_t)) return __builtin_fmaf(static_cast<float>(x), one, -m);
  else return to_f32(x) - m;
}

// V consecutive fp32 values (gamma, beta, saved statistics, partial sums).
template <int V>
__device__ __forceinline__ void load_f32(const float* p, float (&out)[V]) {
  if constexpr (V % 4 == 0) {
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      const F32x4 t = *reinterpret_cast<const F32x4*>(p + i);
      out[i] = t.v[0];
      out[i + 1] = t.v[1];
      out[i + 2] = t.v[2];
      out[i + 3] = t.v[3];
    }
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) out[i] = p[i];
  }
}
template <int V>
__device__ __forceinline__ void load_f32_n(const float* p, float (&out)[V], int cnt) {
  if (cnt == V) {
    load_f32<V>(p, out);
    return;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) out[i] = i < cnt ? p[i] : 0.f;
}
template <int V>
__device__ __forceinline__ void store_f32(float* p, const float (&in)[V]) {
  if constexpr (V % 4 == 0) {
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      *reinterpret_cast<F32x4*>(p + i) = F32x4{{in[i], in[i + 1], in[i + 2], in[i + 3]}};
    }
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) p[i] = in[i];
  }
}

template <int V>
__device__ __forceinline__ void store_f32_n(float* p, const float (&in)[V], int cnt) {
  if (cnt == V) {
    store_f32<V>(p, in);
    return;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (i < cnt) p[i] = in[i];
  }
}

template <int V>
__device__ __forceinline__ void store_f32_from(float* p, const float (&in)[V], int lo) {
  if (lo == 0) {
    store_f32<V>(p, in);
    return;
  }
#pragma unroll
  for (int i = 0; i < V; ++i) {
    if (i >= lo) p[i] = in[i];
  }
}

// ------------------------------------------------------------------ cross-lane
// Exchange with the lane whose id differs in bit `mask` (true butterfly step; goes
// through the LDS crossbar, so it is kept off the per-row paths).
__device__ __forceinline__ float lane_xor(float v, int mask) { return __shfl_xor(v, mask, kWave); }

// DPP controls (gfx9 encoding).
constexpr int kDppQuadXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <-> 7 - i inside each 8 lanes
constexpr int kDppRowMirror = 0x140;      // lane i <-> 15 - i inside each 16 lanes

template <int CTRL>
__device__ __forceinline__ float dpp_read(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// v + (v of the sibling 16-lane row / 32-lane half) through v_permlane{16,32}_swap_b32.
// The instruction swaps the odd rows (upper half) of its first register with the even rows
// (lower half) of its second; fed two copies of v, the first register ends up holding the
// even-row (lower-half) values everywhere and the second the odd-row (upper-half) values,
// so their sum is the pair total in every lane.  The second copy goes through an empty
// asm so that the compiler treats the two results as distinct values.
template <int SPAN>
__device__ __forceinline__ float swap_add(float v) {
  const unsigned a = __builtin_bit_cast(unsigned, v);
  unsigned b = a;
  asm volatile("" : "+v"(b));
  unsigned r0, r1;
  if constexpr (SPAN == 16) {
    auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
    r0 = r[0];
    r1 = r[1];
  } else {
    auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
    r0 = r[0];
    r1 = r[1];
  }
  return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

// All-reduce (sum) over aligned groups of WIDTH lanes, WIDTH a power of two <= 64, with
// VALU cross-lane operations only: two quad permutes, the two row mirrors, then the
// gfx950 v_permlane16_swap / v_permlane32_swap for the 32- and 64-lane steps.  The
// mirrors are not butterflies, but every lane of a sub-group already holds the
// sub-group's total when they are applied, so pairing with ANY lane of the sibling
// sub-group is enough.  Additions are commutative, so every lane of the group ends with
// the same bits.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(WIDTH >= 1 && WIDTH <= 64 && (WIDTH & (WIDTH - 1)) == 0, "bad width");
  if constexpr (WIDTH >= 2) v += dpp_read<kDppQuadXor1>(v);
  if constexpr (WIDTH >= 4) v += dpp_read<kDppQuadXor2>(v);
  if constexpr (WIDTH >= 8) v += dpp_read<kDppRowHalfMirror>(v);
  if constexpr (WIDTH >= 16) v += dpp_read<kDppRowMirror>(v);
  if constexpr (WIDTH >= 32) v = swap_add<16>(v);
  if constexpr (WIDTH >= 64) v = swap_add<32>(v);
  return v;
}

// ---------------------------------------------------- values exchanged between workgroups
// Workgroups of one launch that hand each other partial results through memory while they run
// (the single-launch channels-last kernels, the channel-first backward's fold over the batch)
// write every value as an 8-byte word (value, tag) with one store.  The tag is a number that
// no earlier call of the process has used, so a word either still carries an older call's tag
// or is complete: no separate flag, no fence, nothing to clear between calls.  Values travel in
// pairs; the second word carries the complemented tag, so 64 bits of arbitrary memory would
// have to match before garbage in a fresh workspace could pass for data.  Readers poll with
// device-scope loads, which never return a stale cache line, a bounded number of times.
typedef unsigned long long cl_word;

__device__ __forceinline__ cl_word cl_tagged(float v, unsigned tag) {
  return static_cast<cl_word>(__builtin_bit_cast(unsigned, v)) | (static_cast<cl_word>(tag) << 32);
}
__device__ __forceinline__ cl_word cl_peek(const cl_word* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// A pair of tagged words as one 16-byte store (each aligned 8-byte half lands whole).
__device__ __forceinline__ void cl_publish(cl_word* pair, float a, float b, unsigned tag) {
  typedef cl_word w2 __attribute__((ext_vector_type(2)));
  w2 v;
  v.x = cl_tagged(a, tag);
  v.y = cl_tagged(b, ~tag);
  *reinterpret_cast<w2*>(pair) = v;
}
// The same, written through to memory (readers on other XCDs).
__device__ __forceinline__ void cl_publish_device(cl_word* pair, float a, float b, unsigned tag) {
  __hip_atomic_store(pair, cl_tagged(a, tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(pair + 1, cl_tagged(b, ~tag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One round of a wave's wait for the pair at `pair` (per lane; lanes with want == false wait for
// nothing): reads both words and tells whether every wanted lane found this call's tag in both.
// All 64 lanes of the wave must call it; the result is the same in all of them.
__device__ __forceinline__ bool cl_try_pair(const cl_word* pair, bool want, unsigned tag, float& a, float& b) {
  bool ready = true;
  if (want) {
    const cl_word w0 = cl_peek(pair);
    const cl_word w1 = cl_peek(pair + 1);
    ready = static_cast<unsigned>(w0 >> 32) == tag && static_cast<unsigned>(w1 >> 32) == ~tag;
    a = __builtin_bit_cast(float, static_cast<unsigned>(w0));
    b = __builtin_bit_cast(float, static_cast<unsigned>(w1));
  }
  return __all(ready);
}
// The wait itself: true once a round succeeds, false after max_polls rounds.
__device__ __forceinline__ bool cl_wait_pair(const cl_word* pair, bool want, unsigned tag, int max_polls,
                                             float& a, float& b) {
  a = b = 0.f;
  for (int poll = 0; poll < max_polls; ++poll) {
    if (cl_try_pair(pair, want, tag, a, b)) return true;
  }
  return false;
}

// How patient the waits of a call are.  The kernels whose workgroups exchange results need the
// workgroups of one instance / plane resident together; where another kernel fills whole CUs they
// never are, every wait runs out, and what costs the time is the waiting (the workgroups that give
// up do the missing work between them).  `trouble` is a word of device memory that holds the tag
// of the last call in which a patient wait ran out.  A wait polls kExchangeHastyPolls times
// first, which is mostly enough when the peers are resident; only then does it read the word (a
// call on a GPU of its own seldom touches it).  For kExchangeTroubleCalls calls after the one
// recorded there it gives up at once, which costs a little redundant work when the peers were
// merely slow; after that a call waits patiently again and finds out whether the GPU is still
// shared.  Results do not depend on any of this (whatever a workgroup computes for a peer has the
// peer's bits).
constexpr int kExchangePatientPolls = 100;  // poll limits from here on count as patient
constexpr int kExchangeHastyPolls = 24;
constexpr unsigned kExchangeTroubleCalls = 256;
// cl_wait_pair under that rule.  All 64 lanes of the wave must call it; the result is the same
// in all of them.  trouble == nullptr or a limit below kExchangePatientPolls: the plain wait.
__device__ __forceinline__ bool exchange_wait_pair(const cl_word* pair, bool want, unsigned tag, int max_polls,
                                                   unsigned* trouble, float& a, float& b) {
  a = b = 0.f;
  const bool adaptive = trouble != nullptr && max_polls >= kExchangePatientPolls;
  for (int poll = 0; poll < max_polls; ++poll) {
    // (the record is fetched along with the poll's own loads: one round trip, not two)
    const bool decide = adaptive && poll == kExchangeHastyPolls - 1;
    unsigned seen = 0;
    if (decide) seen = __hip_atomic_load(trouble, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (cl_try_pair(pair, want, tag, a, b)) return true;
    if (decide && tag - seen < kExchangeTroubleCalls) return false;
  }
  if (adaptive && (threadIdx.x & (kWave - 1)) == 0) {
    __hip_atomic_store(trouble, tag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  return false;
}

// Loops over strided indices are written in batches of B whose loads are all issued before
// the first is consumed: the compiler does not move a load above the bounds check of the
// iteration before it, so a plain loop would pay one memory latency per iteration.
template <int B, typename Full, typename Tail>
__device__ __forceinline__ void batched_for(int64_t first, int64_t end, int64_t step, Full&& full,
                                            Tail&& tail) {
  int64_t p = first;
  for (; p + (B - 1) * step < end; p += B * step) full(p, step);
  for (; p < end; p += step) tail(p);
}
// Fast reciprocal (v_rcp_f32, 1 ulp): used for counts, which are small integers.
__device__ __forceinline__ float fast_rcp(float v) { return __builtin_amdgcn_rcpf(v); }

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
  const float inv = r.n > 0.f ? fast_rcp(r.n) : 0.f;
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

// blockDim.x.  Kernels read it once at their start and hand the value (or the wave count) to the
// helpers below, so that no helper called inside a loop reads the block size itself: such a read
// can end up as a load from the dispatch packet in the loop, whose wait also waits for every
// prefetch issued before it.  (Hiding the value from the optimiser behind an empty asm
// statement, to rule that out entirely, cost the block-per-row forward 10-20 %: the compiler
// uses what it knows about the block size.)
__device__ __forceinline__ int block_threads() { return static_cast<int>(blockDim.x); }

// Block-wide Welford all-reduce for blocks that are a whole number of waves (nw of them).
// `buf` must hold 16 Wf entries and be private to this call until the block has passed
// another barrier (callers alternate between two buffers).
__device__ __forceinline__ Wf block_wf(Wf w, Wf* buf, int nw) {
  w = group_wf<kWave>(w);
  if (nw == 1) return w;
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = w;
  __syncthreads();
  Wf r = buf[0];
  for (int i = 1; i < nw; ++i) r = wf_merge(r, buf[i]);
  return r;
}

// Block-wide all-reduce of two sums, same contract as block_wf (`buf` holds 16 float2).
__device__ __forceinline__ float2 block_sum2(float a, float b, float2* buf, int nw) {
  a = group_sum<kWave>(a);
  b = group_sum<kWave>(b);
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

// All-reduce of two sums over each group of WPG consecutive waves of the block (a row held
// by WPG * 64 threads); same buffer contract as block_sum2.  Every wave of the block must
// call it (it contains a block-wide barrier).
template <int WPG>
__device__ __forceinline__ float2 wavegroup_sum2(float a, float b, float2* buf) {
  a = group_sum<kWave>(a);
  b = group_sum<kWave>(b);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = make_float2(a, b);
  __syncthreads();
  const int first = wave / WPG * WPG;
  float2 r = buf[first];
#pragma unroll
  for (int i = 1; i < WPG; ++i) {
    r.x += buf[first + i].x;
    r.y += buf[first + i].y;
  }
  return r;
}

// Block-wide all-reduce of one sum, same contract (`buf` holds 16 floats).
__device__ __forceinline__ float block_sum1(float a, float* buf, int nw) {
  a = group_sum<kWave>(a);
  if (nw == 1) return a;
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = a;
  __syncthreads();
  float r = buf[0];
  for (int i = 1; i < nw; ++i) r += buf[i];
  return r;
}

// Streaming statistics without a pivot: a thread takes its values in small register-resident
// batches, gets each batch's (mean, m2) by an exact two-pass over the registers and merges it
// into its running triple with Chan's update (reference: norm_util.h:190-210, whose per-element
// push is the batch-of-one case).  No term is a difference of large sums, so an outlier
// anywhere in the data costs no precision; per element it is one add, one subtract and one
// FMA, the merge (a reciprocal and ten operations) is shared by the whole batch.
__device__ __forceinline__ void wf_push_batch(Wf& run, float batch_mean, float batch_m2, float nb) {
  const float n = run.n + nb;
  const float w = nb * fast_rcp(n);
  const float d = batch_mean - run.mean;
  run.m2 += batch_m2 + (d * d) * (run.n * w);
  run.mean += d * w;
  run.n = n;
}
template <int N>
__device__ __forceinline__ void wf_push(Wf& run, const float (&f)[N]) {
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) s += f[i];
  const float mb = s * (1.0f / N);
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = f[i] - mb;
    q += d * d;
  }
  wf_push_batch(run, mb, q, static_cast<float>(N));
}

// The same for V independent streams that advance together (the V channels of a thread's
// channel vector): one count, one reciprocal per batch.
template <int V>
struct WfLanes {
  float mean[V], m2[V];
  float n;
};
template <int V>
__device__ __forceinline__ void wf_lanes_init(WfLanes<V>& w) {
#pragma unroll
  for (int i = 0; i < V; ++i) w.mean[i] = w.m2[i] = 0.f;
  w.n = 0.f;
}
// f[u][i]: value u of stream i; all B values of every stream are valid.
template <int V, int B>
__device__ __forceinline__ void wf_lanes_push(WfLanes<V>& run, const float (&f)[B][V]) {
  const float n = run.n + static_cast<float>(B);
  const float w = static_cast<float>(B) * fast_rcp(n);
  const float cross = run.n * w;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < B; ++u) s += f[u][i];
    const float mb = s * (1.0f / B);
    float q = 0.f;
#pragma unroll
    for (int u = 0; u < B; ++u) {
      const float d = f[u][i] - mb;
      q += d * d;
    }
    const float d = mb - run.mean[i];
    run.m2[i] += q + (d * d) * cross;
    run.mean[i] += d * w;
  }
  run.n = n;
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
