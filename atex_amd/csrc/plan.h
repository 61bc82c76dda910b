// Host-side launch planning: which kernel family, which geometry and how much workspace
// a call needs.  Pure host code with no HIP dependency, shared by the launchers and by
// the *_workspace_bytes queries so that both always agree.
//
// It plays the part of the reference's dispatch ladders
// (fused_layer_norm_op.cu:824-891, :919-1028; fused_instance_norm_op.cu:1203-1561) but
// decides from row length, row count and the CU count instead of from occupancy probes
// against a 48 KB shared-memory limit.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <algorithm>
#include <atomic>
#include <climits>

namespace atexn {

// Launch-planning parameters; the defaults were chosen by measurement on MI355X.  In the
// product library they are constants: it keeps no process-wide state, and a workspace query and
// the call it sizes always see the same plan.  Only the benchmark build of the library
// (-DATEXN_BENCH_BUILD, libatex_norms_hip_bench.so) can change them, through atexn_set_tuning,
// for A/B measurements and for tests that force a particular kernel family; there each is an
// atomic so that a change made while other threads plan launches is a clean switch.
#ifdef ATEXN_BENCH_BUILD
using TuneInt = std::atomic<int>;
#else
struct TuneInt {
  int v;
  constexpr TuneInt(int x) : v(x) {}
  constexpr int load() const { return v; }
  constexpr operator int() const { return v; }
};
#endif
struct Tuning {
  TuneInt fwd_waves_per_cu{16};      // resident forward: waves kept resident per CU
  TuneInt bwd_ln_threads{512};       // resident LayerNorm backward, rows <= one wave: block size
  TuneInt bwd_waves_per_cu{8};       // resident LayerNorm backward: waves kept resident per CU
                                     //   (each block adds a partial row to the column reduction)
  TuneInt bwd_affine_waves_per_cu{32};  // resident channel-first backward (no partial rows)
  TuneInt split_items_per_cu{2};     // split rows: (row, chunk) work items per CU, forward
  TuneInt split_bwd_items_per_cu{4};  //   and backward
  TuneInt cl_items_per_cu{2};        // channels-last: (n, slab, tile) work items per CU
  TuneInt cl_bwd_big_items{1};       //   the same for the backward of tensors of 2^25 elements and more
  TuneInt tile_items_per_cu{4};      // LayerNorm long rows: (row slab, column tile) tiles per CU
  TuneInt fwd_rows_batch{4};         // resident kernels, rows <= one wave: rows per batch of a
  TuneInt fwd_rows_batch_v1{1};      //   (forward with one vector per lane)
  TuneInt bwd_rows_batch{2};         //   lane group (fwd 1, 2, 4; bwd 1, 2; vector path only)
  TuneInt staged_rows{1};            // rows beyond the registers staged in LDS, single pass (0: never, 2: however few rows)
  TuneInt bwd_lds_vpt{4};            //   its vectors per lane: 4 (up to 640 / 1024 threads) or 8 (up to 512)
  TuneInt bwd_lds_rows{1};           // LayerNorm backward: the single-pass kernel with accumulators in LDS
  TuneInt bwd_min_rows{4};           // resident LayerNorm backward: rows per workgroup worth a partial row
  // Two-stage kernels: stage 2 walks its chunk / slab from the end (what stage 1 touched last
  // is what the memory-side cache still holds).
  TuneInt reverse_second_pass{1};
  TuneInt cl_narrow_tiles{1};   // channels-last two-stage kernels: tiles of 8 channel vectors when pixels are line-aligned
  TuneInt cl_fold_cap{1};     // channels-last: no more slabs than a stage-2 fold takes from registers
  TuneInt cl_fused_split{1};  // channels-last single pass: narrower channel tiles so that an instance fits
  TuneInt cl_fused{1};        // channels-last: single-pass kernels when an instance fits a workgroup
  // channels-last: statistics and their use in one launch (cl_single_kernels.hip.h) when every
  // slab is register-resident and all workgroups fit the chip at once; and how many polls a wait
  // for a peer's partials may take before a workgroup recomputes them itself (0: at once)
  TuneInt cl_single{1};
  TuneInt cl_single_xm{1};  //   also on the XCD-major grid (any batch size, any number of workgroups)
  TuneInt cl_single_occ{1};  //   on that grid, when the launch does not fit the chip: the kernels compiled for more workgroups per CU
  TuneInt cl_single_polls{300};
  TuneInt affine_fold{1};      // channel-first backward, a workgroup per plane: dgamma / dbeta folded over the batch in the row kernel
  TuneInt affine_fold_polls{2000};  //   polls before a workgroup recomputes its peers' plane sums (0: at once)
  // channel-first planes too long for a workgroup: the chunks of a plane on the workgroups of one
  // XCD, statistics exchanged while they run, one pass (plane_single_kernels.hip.h); and its polls
  TuneInt plane_single{1};
  TuneInt plane_single_polls{500};
  // 1: plane_bwd_single built for three workgroups per CU when a plane has more than 32 chunks
  TuneInt plane_single_occ{1};
  TuneInt plane_nt_min_mb{256};  // forward: non-temporal loads of x from this many MiB (what no cache level retains anyway)
  TuneInt bwd_wave_groups{1};  // LayerNorm backward, 129..512 vectors per row: rows on 2 / 4 waves
  // Block-wide resident rows: longest row (in vectors) that uses 2 vectors per thread (more,
  // smaller-register threads) before switching to 4; forward <= 2048, backward <= 1536.
  TuneInt fwd_vpt2_max_vec{1536};    // LayerNorm forward, a workgroup per row: 2 vectors per lane up to this many vectors (768 threads)
  TuneInt bwd_vpt2_max_vec{1536};
  TuneInt fwd_vpt4_max_vec{3072};    // LayerNorm forward, a workgroup per row: 4 vectors per lane up to this many vectors (768 threads)
#ifdef ATEXN_BENCH_BUILD
  // Only in the benchmark build of the library (libatex_norms_hip_bench.so): which stages of a
  // backward call over resident rows run (bit 0: the row kernel, bit 1: the column reduction),
  // so that the row kernel can be timed alone.  Anything but 3 gives incomplete results, which
  // is why the product library has no such switch.
  TuneInt bwd_stage_mask{3};
#endif
};
#ifdef ATEXN_BENCH_BUILD
Tuning& tuning();
#else
const Tuning& tuning();
#endif
inline int bwd_stage_mask() {
#ifdef ATEXN_BENCH_BUILD
  return tuning().bwd_stage_mask;
#else
  return 3;
#endif
}

constexpr int kPlanXcdCount = 8;  // workgroups are dealt to the XCDs of an MI355X in turn
enum class RowsKind { kFwd, kBwdCols /*LayerNorm: per-column dgamma/dbeta*/, kBwdAffine };

inline int64_t div_up(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int64_t round_up(int64_t a, int64_t b) { return div_up(a, b) * b; }
inline size_t align256(size_t b) { return (b + 255) & ~static_cast<size_t>(255); }
inline int pow2_ceil(int64_t v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

struct RowsPlan {
  int V = 1;  // storage elements per access
  bool resident = false;
  // resident
  int tpr = 0, vpt = 1, threads = 256, rpb = 1, rb = 1;
  bool exact = false;  // no lane, vector or row of any batch falls outside the data
  bool ragged = false;  // D % V != 0: the last vector of a row is partial
  int grid = 1;
  size_t fold_lds = 0;  // dynamic LDS of the LayerNorm backward fold
  bool acc_lds = false;  // LayerNorm backward with the column accumulators in LDS (rows_bwd_lds)
  bool staged = false;   // single pass with the row staged in registers + LDS (rows_*_staged)
  int nv_lds = 0;        //   vectors per thread kept in LDS (the first 8 stay in registers)
  // split
  int S = 1;
  int64_t chunk = 0;
  int split_grid = 1;
  // workspace sections (bytes from the start of the workspace)
  size_t off_part = 0, off_pairs = 0, ws_bytes = 0;
  int part_rows = 0;  // G of the column reduction
  // Channel-first backward with a workgroup per plane: the fold of the plane sums over the batch
  // runs inside the row kernel (tagged pairs at off_tagged, 16 bytes per plane) instead of as a
  // col_reduce launch.  Needs the planes of a channel on one XCD (C and the grid multiples of the
  // XCD count), the grid a multiple of C or C of the grid, at most 64 instances; the launcher
  // also wants dx != dy and no stream capture.
  bool affine_fold = false;
  size_t off_tagged = 0;
  // Channel-first planes beyond the resident and staged kernels, one launch and one pass
  // (plane_single_kernels.hip.h): ps_S chunks of ps_chunk_vec vectors per plane, each on a
  // 512-thread workgroup with at most 8 vectors per thread; workgroup b of the ps_grid takes chunk
  // (b / 8) % ps_S of plane ((b / 8) / ps_S) * 8 + b % 8.  Needs whole vectors (D % V == 0) and no
  // more chunks than an XCD holds such workgroups (two per CU).  The split kernels stay the
  // fallback (y == x, stream capture) in the same workspace; tagged pairs at off_ps_tagged.
  bool plane_single = false;
  int ps_S = 0, ps_chunk_vec = 0, ps_grid = 0;
  bool ps_full = false;  // every thread of every workgroup holds 8 vectors
  size_t off_ps_tagged = 0;
  size_t off_ps_claims = 0;  // a word per chunk: who computes it when its workgroup is not there
  // backward: the planes' sums folded over the batch inside the kernel (tagged pairs per plane at
  // off_ps_fold) instead of by a col_reduce launch: the planes of a channel must share an XCD (C a
  // multiple of the XCD count, or a single instance), at most 64 instances
  bool ps_fold = false;
  size_t off_ps_fold = 0;
};
constexpr int kPlanAffineFoldMaxStep = 64, kPlanAffineFoldMaxPairs = 1024;
constexpr int kPlanPlaneThreads = 512, kPlanPlaneVpt = 8, kPlanPlaneMaxChunks = 64;

// Longest row, in vectors, that the register-resident kernels take: forward 8 vectors per
// thread at 512 threads, backward 4 (it holds x and dy, and LayerNorm also gamma and the
// dgamma / dbeta accumulators of its columns).
// The channel-first InstanceNorm backward has no such accumulators and goes as far as the
// forward.
inline int64_t resident_limit(RowsKind kind) { return kind == RowsKind::kBwdCols ? 2048 : 4096; }

// LayerNorm backward beyond that: one more single-pass kernel keeps the dgamma / dbeta
// accumulators of a workgroup's columns in LDS (rows_bwd_lds: 8 bytes per column, 8 vectors per
// thread at up to 512 threads) while they fit the 160 KiB of a gfx950 CU beside the block
// reductions' buffer.
constexpr size_t kPlanLdsBytes = 160 * 1024;
constexpr size_t kPlanBwdLdsReserve = 512;
inline size_t bwd_lds_bytes(int64_t D) { return size_t(round_up(D, 4)) * 2 * sizeof(float); }
// Rows staged on chip (rows_fwd_staged / rows_bwd_staged): 512 threads, 8 vectors per thread in
// registers and the rest in LDS (16 bytes per vector forward, 32 backward: x and dy).
constexpr int kPlanStagedThreads = 512;
constexpr int kPlanStagedRegVec = 8;
inline int staged_lds_vectors(RowsKind kind, int64_t n_vec) {
  return static_cast<int>(std::max<int64_t>(0, div_up(n_vec, kPlanStagedThreads) - kPlanStagedRegVec));
}
inline size_t staged_lds_bytes(RowsKind kind, int64_t n_vec) {
  return size_t(staged_lds_vectors(kind, n_vec)) * kPlanStagedThreads * (kind == RowsKind::kFwd ? 16 : 32);
}
// One workgroup streams a row at a few tens of GB/s (its loads in flight over the memory
// latency), so staging pays once there are enough rows to keep every CU busy for several of
// them: measured against the two-stage kernels, [1024, 65536] fp16 planes 65 / 111 -> 53 / 93 us,
// but 256 such planes 16.8 -> 20.9 us forward (backward 28.4 -> 26.3 us) and a single one twice as slow.
inline bool staged_fits(RowsKind kind, int V, int64_t n_rows, int64_t D, int cus) {
  return V > 1 && kind != RowsKind::kBwdCols && tuning().staged_rows && D < (int64_t(1) << 31) &&
         (tuning().staged_rows == 2 || n_rows >= int64_t(cus) * (kind == RowsKind::kFwd ? 2 : 1)) &&
         staged_lds_bytes(kind, div_up(D, V)) + kPlanBwdLdsReserve <= kPlanLdsBytes;
}
inline bool bwd_lds_fits(int V, int64_t D) {
  return V > 1 && tuning().bwd_lds_rows && div_up(D, V) <= 4096 && bwd_lds_bytes(D) + kPlanBwdLdsReserve <= kPlanLdsBytes;
}

// Which kernels take a contiguous-row problem.  vec = 16 / sizeof(T).
//   V = vec: rows of at least one vector (a ragged end, D % vec != 0, is handled inside the
//            kernels); V = 1: rows shorter than a vector;
//   tiles:   LayerNorm rows beyond the resident limit (any D).
//   small:   rows of at most 4 vectors when there are many of them: one thread per row.
struct RowsRoute {
  int V = 1;
  bool tiles = false;
  bool small = false;
};
// LDS of the LayerNorm backward's fold: same constants as rows_kernels.hip.h
constexpr int kPlanFoldLdsBytes = 64 * 1024;
constexpr int kPlanFoldMaxWaves = 8;
constexpr int kPlanSmallMaxVec = 4;
constexpr int64_t kPlanSmallMinRows = 4096;
inline RowsRoute route_rows(RowsKind kind, bool layer_norm, int vec, int64_t n_rows, int64_t D) {
  RowsRoute r;
  if (D >= vec && div_up(D, vec) <= kPlanSmallMaxVec && n_rows >= kPlanSmallMinRows) {
    r.V = vec;
    r.small = true;
    return r;
  }
  if (D >= vec) r.V = vec;  // ragged row ends are handled by every vector kernel
  r.tiles = layer_norm && div_up(D, r.V) > resident_limit(kind) &&
            !(kind == RowsKind::kBwdCols && bwd_lds_fits(r.V, D));
  return r;
}

struct SmallPlan {
  int NV = 1;
  int grid = 1;
  int part_rows = 0;
  size_t ws_bytes = 0;
};
inline SmallPlan plan_small(RowsKind kind, int V, int64_t n_rows, int64_t D, int C, int cus) {
  SmallPlan p;
  p.NV = static_cast<int>(div_up(D, V));
  p.grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(div_up(n_rows, 256), int64_t(cus) * 8)));
  if (kind == RowsKind::kBwdCols) {
    p.part_rows = p.grid;
    p.ws_bytes = align256(sizeof(float) * 2 * size_t(D) * size_t(p.grid));
  } else if (kind == RowsKind::kBwdAffine) {
    p.part_rows = static_cast<int>(n_rows / C);
    p.ws_bytes = align256(sizeof(float) * 2 * size_t(n_rows));
  }
  return p;
}

// Adds the one-launch plan for channel-first planes (RowsPlan::plane_single) to a plan whose other
// workspace sections end at `bytes`, when the shape qualifies.
inline void plan_plane_single(RowsPlan& p, RowsKind kind, int V, int64_t n_rows, int64_t D, int C, int cus,
                              size_t& bytes) {
  const Tuning& t = tuning();
  const int64_t n_vec = div_up(D, V);
  if (t.plane_single && C > 0 && V > 1 && D % V == 0 && kind != RowsKind::kBwdCols) {
    const int64_t per_wg = int64_t(kPlanPlaneThreads) * kPlanPlaneVpt;
    const int64_t S2 = div_up(n_vec, per_wg);
    const int64_t slots = int64_t(cus / kPlanXcdCount) * 2;
    const int64_t grid = round_up(n_rows, kPlanXcdCount) * S2;
    if (S2 >= 2 && S2 <= std::min<int64_t>(kPlanPlaneMaxChunks, slots) && grid < (int64_t(1) << 31)) {
      p.plane_single = true;
      p.ps_S = static_cast<int>(S2);
      p.ps_chunk_vec = static_cast<int>(div_up(n_vec, S2));
      p.ps_grid = static_cast<int>(grid);
      p.ps_full = n_vec % S2 == 0 && p.ps_chunk_vec == per_wg;
      p.off_ps_tagged = bytes;
      bytes += align256(size_t(16) * size_t(n_rows) * size_t(S2));
      p.off_ps_claims = bytes;
      bytes += align256(size_t(4) * size_t(n_rows) * size_t(S2));
      if (kind == RowsKind::kBwdAffine && t.affine_fold && p.part_rows <= 64 &&
          (C % kPlanXcdCount == 0 || p.part_rows == 1)) {
        p.ps_fold = true;
        p.off_ps_fold = bytes;
        bytes += align256(size_t(16) * size_t(n_rows));
      }
    }
  }
}

// V: vector width in elements (see route_rows).  C: the channel count of a channel-first input
// (row r takes gamma[r % C]), 0 for LayerNorm.
inline RowsPlan plan_rows(RowsKind kind, int V, int64_t n_rows, int64_t D, int C, int cus) {
  const Tuning& t = tuning();
  RowsPlan p;
  p.V = V;
  const int64_t n_vec = div_up(D, V);
  p.ragged = D % V != 0;
  p.resident = n_vec <= resident_limit(kind);
  if (!p.resident && kind == RowsKind::kBwdCols && bwd_lds_fits(V, D)) {
    p.resident = true;
    p.acc_lds = true;
    p.tpr = 0;
    p.vpt = t.bwd_lds_vpt;
    p.threads = static_cast<int>(round_up(div_up(n_vec, p.vpt), 64));
    p.rpb = 1;
    p.rb = 1;
    p.fold_lds = bwd_lds_bytes(D);
    p.grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(n_rows, cus)));  // one workgroup per CU (LDS)
    while (p.grid >= cus && p.grid > 1 && div_up(n_rows, p.grid) < t.bwd_min_rows) p.grid = (p.grid + 1) / 2;
    p.part_rows = p.grid;
    p.off_part = 0;
    p.ws_bytes = align256(sizeof(float) * 2 * size_t(D) * size_t(p.grid));
    return p;
  }
  if (!p.resident && staged_fits(kind, V, n_rows, D, cus)) {
    p.staged = true;
    p.threads = kPlanStagedThreads;
    p.nv_lds = staged_lds_vectors(kind, n_vec);
    p.fold_lds = staged_lds_bytes(kind, n_vec);
    // workgroups per CU: what the LDS leaves room for, at most four (2048 threads)
    const int64_t per_cu = std::max<int64_t>(1, std::min<int64_t>(4, int64_t(kPlanLdsBytes) / int64_t(p.fold_lds + kPlanBwdLdsReserve)));
    p.grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(n_rows, int64_t(cus) * per_cu)));
    if (kind == RowsKind::kBwdAffine) {
      p.part_rows = static_cast<int>(n_rows / C);
      p.off_part = 0;
      p.ws_bytes = align256(sizeof(float) * 2 * size_t(n_rows));
    }
    // (the one-launch kernels over the workgroups of an XCD, where they apply, are faster:
    // [16, 64, 256, 256] fp16 44.7 / 86.1 us staged, 41.9 / 74.8 us so; the staged kernels then
    // serve y == x, stream capture and ragged planes)
    plan_plane_single(p, kind, V, n_rows, D, C, cus, p.ws_bytes);
    return p;
  }
  if (p.resident) {
    // Rows of up to 192 vectors sit on a group of 8..64 lanes with 1, 2 or 3 vectors per lane:
    // the candidate with the fewest slots wins (3 vectors per lane make the 3 * 2^k hidden
    // sizes, 768, 1536, ..., exact), ties go to fewer vectors per lane.
    int64_t best_slots = INT64_MAX;
    if (V > 1 || n_vec <= 8) {
      for (int vpt = 1; vpt <= (V > 1 ? 3 : 1); ++vpt) {
        const int tpr = std::max(8, pow2_ceil(div_up(n_vec, vpt)));
        if (tpr > 64 || (vpt == 2 && tpr != 64)) continue;
        if (int64_t(tpr) * vpt < best_slots) {
          best_slots = int64_t(tpr) * vpt;
          p.tpr = tpr;
          p.vpt = vpt;
        }
      }
    }
    if (best_slots != INT64_MAX) {
      // chosen above
    } else if (kind == RowsKind::kBwdCols && V > 1 && n_vec <= 512 && t.bwd_wave_groups &&
               n_rows >= int64_t(cus) * (n_vec <= 256 ? 4 : 2)) {
      // LayerNorm backward: 512-thread blocks with 2 or 4 waves per row, so that a block
      // still covers several rows (one dgamma / dbeta partial row per block)
      p.tpr = n_vec <= 256 ? 128 : (n_vec <= 384 ? 128 : 256);
      p.vpt = n_vec <= 256 ? 2 : (n_vec <= 384 ? 3 : 2);
    } else {
      p.tpr = 0;
      // (the LayerNorm forward takes fewer vectors per lane on more threads further up than the
      // channel-first one, here and below: [4092, 8200] halves 30.5 -> 22.9 us with 2 per lane,
      // planes of 9000 .. 12288 halves 3 % slower)
      const int vpt2_max = kind == RowsKind::kFwd ? (C == 0 ? t.fwd_vpt2_max_vec.load() : 1024) : t.bwd_vpt2_max_vec.load();
      // LayerNorm forward: 4 vectors per lane on up to 768 threads beat 8 on 512 ([2048, 20480]
      // halves 35 -> 28 us); channel-first planes of that size, with no gamma / beta vectors
      // to read, are faster with the 8 loads per lane in flight, and so is every backward
      const int vpt4_max = kind == RowsKind::kFwd && C == 0 ? t.fwd_vpt4_max_vec.load() : 2048;
      p.vpt = n_vec <= vpt2_max ? 2 : (n_vec <= vpt4_max ? 4 : 8);
    }
    if (p.tpr > 64) {
      p.threads = 512;
      p.rpb = p.threads / p.tpr;
    } else if (p.tpr == 0) {
      p.threads = static_cast<int>(round_up(div_up(n_vec, p.vpt), 64));
      p.rpb = 1;
    } else {
      p.threads = 256;
      if (V > 1 && (!p.ragged || p.vpt == 1)) {
        // backward: two rows per batch pay for rows of one vector per lane (D <= 512 halves:
        // 85 -> 89 % of the streaming rate); with more vectors per lane they cost registers
        // and measured slower
        // forward: as many rows per batch as still leave the next batch prefetched (4 vectors per
        // lane in flight: [16384, 1024] halves 12.1 -> 11.1 us with 2 rows of 2 vectors against 4)
        // (and with one vector per lane a single row per batch, the next one prefetched, beats
        // four: [262144, 128] 21.6 -> 20.9 us, [1000000, 100] 84 -> 77 us)
        const int fwd_rb = p.vpt == 1 ? t.fwd_rows_batch_v1.load()
                                      : std::min(t.fwd_rows_batch.load(), std::max(1, 4 / p.vpt));
        p.rb = kind == RowsKind::kFwd ? fwd_rb : (p.vpt == 1 ? t.bwd_rows_batch.load() : 1);
      }
      if (kind == RowsKind::kBwdCols) {
        // bigger blocks -> fewer partial rows for the column reduction
        int th = std::min<int>(t.bwd_ln_threads, 512);
        while (th > 256 && div_up(n_rows, int64_t(th / p.tpr) * p.rb) < cus) th /= 2;
        p.threads = th;
      }
      p.rpb = p.threads / p.tpr;
      while (p.rb > 1 && div_up(n_rows, int64_t(p.rpb) * p.rb) < cus) p.rb /= 2;
    }
    const int64_t groups = div_up(n_rows, int64_t(p.rpb) * p.rb);
    p.exact = V > 1 && !p.ragged && n_vec == int64_t(p.tpr == 0 ? p.threads : p.tpr) * p.vpt &&
              n_rows % (int64_t(p.rpb) * p.rb) == 0;
    const int waves = p.threads / 64;
    const int per_cu = std::max(
        1, (kind == RowsKind::kFwd        ? t.fwd_waves_per_cu
            : kind == RowsKind::kBwdCols ? t.bwd_waves_per_cu
                                         : t.bwd_affine_waves_per_cu) /
               waves);
    p.grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(groups, int64_t(cus) * per_cu)));
    if (kind == RowsKind::kBwdCols) {
      // A workgroup leaves one partial row of 2 * D floats however few rows it had: with fewer
      // than bwd_min_rows (4) rows each, the partial rows are more traffic than the rows.  Few
      // long rows get fewer workgroups (not below half the CUs).
      while (p.grid >= cus && p.grid > 1 && div_up(n_rows, p.grid) < t.bwd_min_rows) p.grid = (p.grid + 1) / 2;
      p.part_rows = p.grid;
      p.off_part = 0;
      p.ws_bytes = align256(sizeof(float) * 2 * size_t(D) * size_t(p.grid));
      if (p.tpr != 0) {
        // the fold of the waves' dgamma / dbeta sums (rows_bwd_resident): waves x groups per
        // pass x lanes with sums x floats per group
        const int w = V % 4 == 0 ? 4 : 1;
        const int lr = std::min(p.tpr, 64);
        const int q = 2 * V * p.vpt / w;
        const int cap = kPlanFoldLdsBytes / (kPlanFoldMaxWaves * lr * w * 4);
        p.fold_lds = size_t(waves) * size_t(std::min(q, cap)) * lr * w * sizeof(float);
      }
    } else if (kind == RowsKind::kBwdAffine) {
      p.part_rows = static_cast<int>(n_rows / C);
      p.off_part = 0;
      p.ws_bytes = align256(sizeof(float) * 2 * size_t(n_rows));
      // (grid a multiple of C or C of the grid: the workgroup that folds a channel is then the
      // last-started of those that handle its planes, and waits for none that starts after it)
      p.affine_fold = t.affine_fold && p.tpr == 0 && C % kPlanXcdCount == 0 && p.grid % kPlanXcdCount == 0 &&
                      (p.grid % C == 0 || C % p.grid == 0) && p.part_rows >= 2 && p.part_rows <= 64;
      if (p.tpr != 0) {
        // lane groups per plane: q consecutive planes per workgroup and step; the same conditions
        // on C / q channel groups, and the fallback's LDS (instances x q pairs)
        const int q = p.rpb * p.rb;
        const int64_t cg = C / q;
        p.affine_fold = t.affine_fold && V > 1 && C % q == 0 && cg % kPlanXcdCount == 0 && p.grid % kPlanXcdCount == 0 &&
                        (p.grid % cg == 0 || cg % p.grid == 0) && p.part_rows >= 2 && p.part_rows <= 64 &&
                        q <= kPlanAffineFoldMaxStep && int64_t(p.part_rows) * q <= kPlanAffineFoldMaxPairs;
      }
      if (p.affine_fold) {
        p.off_tagged = p.ws_bytes;
        p.ws_bytes += align256(size_t(16) * size_t(n_rows));
      }
    }
    return p;
  }
  // split rows
  const int64_t gran = int64_t(256) * V;  // one block sweep
  const int items = kind == RowsKind::kFwd ? t.split_items_per_cu.load() : t.split_bwd_items_per_cu.load();
  const int64_t want = div_up(int64_t(cus) * items, std::max<int64_t>(n_rows, 1));
  const int64_t max_s = std::max<int64_t>(1, D / (gran * 4));
  int64_t S = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, max_s), 1024));
  p.chunk = round_up(div_up(D, S), gran);
  p.S = static_cast<int>(div_up(D, p.chunk));
  const int64_t n_work = n_rows * p.S;
  p.split_grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(n_work, int64_t(cus) * 32)));
  p.off_pairs = 0;
  size_t bytes = align256(sizeof(float) * 2 * size_t(n_work));
  if (kind == RowsKind::kBwdAffine) {
    p.part_rows = static_cast<int>(n_rows / C);
    p.off_part = bytes;
    bytes += align256(sizeof(float) * 2 * size_t(n_rows));
  }
  plan_plane_single(p, kind, V, n_rows, D, C, cus, bytes);
  p.ws_bytes = bytes;
  return p;
}

// LayerNorm rows too long for registers: 2-D tiles of R rows x CW columns (tiles_kernels.hip.h).
// The forward statistics still come from the chunked stage 1 of the split path (S chunks).
struct TilePlan {
  int V = 1;
  int64_t CW = 0;  // columns per tile
  int CT = 1;      // column tiles
  int RS = 1;      // row slabs
  int64_t R = 0;   // rows per slab
  // backward sums stage: its own, possibly narrower, tiling
  int sums_vpt = 4;
  int sums_CT = 1, sums_RS = 1;
  int64_t sums_R = 0;
  int S = 1;       // forward: chunks per row of the statistics stage
  int64_t chunk = 0;
  int stats_grid = 1;
  size_t off_pairs = 0, off_rowsum = 0, off_part = 0, ws_bytes = 0;
};

constexpr int kPlanTileThreads = 256;
constexpr int kPlanTileVpt = 4;

inline TilePlan plan_tiles(bool bwd, int V, int64_t n_rows, int64_t D, int cus) {
  const Tuning& t = tuning();
  TilePlan p;
  p.V = V;
  p.CW = int64_t(kPlanTileThreads) * kPlanTileVpt * V;
  p.CT = static_cast<int>(div_up(D, p.CW));
  const int64_t want = div_up(int64_t(cus) * t.tile_items_per_cu, p.CT);
  int64_t rs = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, n_rows), 1024));
  p.R = div_up(n_rows, rs);
  p.RS = static_cast<int>(div_up(n_rows, p.R));
  size_t bytes = 0;
  if (!bwd) {
    const int64_t gran = int64_t(256) * V;
    const int64_t want_s = div_up(int64_t(cus) * t.split_items_per_cu, std::max<int64_t>(n_rows, 1));
    const int64_t max_s = std::max<int64_t>(1, D / (gran * 4));
    const int64_t S = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want_s, max_s), 1024));
    p.chunk = round_up(div_up(D, S), gran);
    p.S = static_cast<int>(div_up(D, p.chunk));
    p.stats_grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(n_rows * p.S, int64_t(cus) * 32)));
    p.off_pairs = 0;
    bytes = align256(sizeof(float) * 2 * size_t(n_rows) * size_t(p.S));
  } else {
    // sums stage: the widest tile whose partial rows (2 * D floats per row slab, written and
    // read back) stay under about 5 % of the bytes of dy and x; the narrowest otherwise
    for (int vpt = 4; vpt >= 1; vpt /= 2) {
      const int64_t cw = int64_t(kPlanTileThreads) * vpt * V;
      const int64_t ct = div_up(D, cw);
      const int64_t want_rs = div_up(int64_t(cus) * t.tile_items_per_cu, ct);
      int64_t rs2 = std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want_rs, n_rows), 1024));
      const int64_t r = div_up(n_rows, rs2);
      rs2 = div_up(n_rows, r);
      p.sums_vpt = vpt;
      p.sums_CT = static_cast<int>(ct);
      p.sums_RS = static_cast<int>(rs2);
      p.sums_R = r;
      if (rs2 == 1 || rs2 * 80 <= n_rows) break;
    }
    p.off_pairs = 0;
    bytes = align256(sizeof(float) * 2 * size_t(n_rows) * size_t(p.sums_CT));
    p.off_rowsum = bytes;
    bytes += align256(sizeof(float) * 2 * size_t(n_rows));
    p.off_part = bytes;
    if (p.sums_RS > 1) bytes += align256(sizeof(float) * 2 * size_t(D) * size_t(p.sums_RS));
  }
  p.ws_bytes = bytes;
  return p;
}

// Channels-last InstanceNorm, x as [N, D, C].
struct ClPlan {
  int V = 1;
  int CV = 1;    // channel vectors per pixel
  int TPP = 1;   // threads per pixel (power of two <= 256)
  int tpp_shift = 0;
  int CT = 1;    // channel tiles
  int S = 1;     // slabs per instance
  int U = 0;     // vectors per thread of a register-resident slab (0: streaming)
  int64_t slab_len = 0;
  int64_t n_work = 0;
  int grid = 1;
  // More slabs per instance than kClFoldAbove (twice that when four or more lanes of a stage-2
  // workgroup share a channel): a small launch between the two stages adds up the slab partials
  // of every instance once (folded[N][2][C]) instead of every stage-2 workgroup doing it for
  // itself.
  bool fold = false;
  bool fused = false;  // one slab per instance and it fits the registers: single-pass kernels
  int fused_u = 0;     //   with fused_u (1, 2, 4, 8 or 16) pixels per thread
  size_t off_a = 0, off_fold = 0, ws_bytes = 0;
  // One launch per direction (cl_single_kernels.hip.h): the workgroups of an instance exchange
  // their slab partials while they run.  Needs every workgroup on the chip at once (two per CU),
  // all workgroups of an instance on one XCD (the instance index is the fastest grid coordinate
  // and workgroups are dealt to the 8 XCDs in turn: N a multiple of 8), at most 64 slabs and 64
  // instances (a lane each in the folds) and tiles of at most 64 channels.  The launcher also
  // wants y != x and a stream that is not being captured; the two-stage kernels stay the
  // fallback, in the same workspace.
  bool single = false;
  size_t off_tagged = 0, off_finals = 0, off_finals_dev = 0;
  size_t off_claims = 0;  // a word per (instance, tile, slab): who computes it when its workgroup is not there
  // The same kernels on a one-dimensional XCD-major grid (cl_single_place) for launches that do
  // not meet the conditions on N and on the number of workgroups: any batch size, any number of
  // instances; an instance's slabs must fit one XCD (two workgroups per CU).  The backward then
  // leaves per-instance sums at off_xm_part for a col_reduce launch (N > 1).
  bool single_xm = false;
  int xm_grid = 0;
  size_t off_xm_part = 0;
  // ... unless every workgroup of the XCD-major grid is on the chip at once after all (whole
  // units per XCD, N <= 64): the fold over the instances then runs in the kernel as on the
  // other grid
  bool xm_fold = false;
  bool xm_resident = false;  // every workgroup of the XCD-major grid on the chip at once
};
constexpr int kClFoldAbove = 64;
constexpr int kPlanClSingleMaxCap = 64, kPlanClSingleMaxSlabs = 64, kPlanClSingleMaxOwned = 4;
// slab partials per lane that a stage-2 fold takes in one round trip (cl_kernels.hip.h: twice
// kClFoldRegs)
constexpr int kPlanClFoldRegs = 32;

// Width (as a shift: 64, 16, 4 or 1 columns) of the chunks of adjacent dgamma / dbeta columns
// that the channels-last backward's stage 2 deals to its workgroups (cl_fold_sums): `rows`
// partial rows of W2 columns, n_blocks workgroups of 256 threads; a chunk is summed by 256 / cw
// thread rows taking four partial rows each per round trip.  The width with the fewest
// dependent round trips per workgroup wins, the wider one on a tie (longer contiguous reads).
inline int cl_dparam_chunk_shift(int64_t rows, int64_t W2, int64_t n_blocks) {
  int best_shift = 0;
  int64_t best = INT64_MAX;
  for (int sh = 6; sh >= 0; sh -= 2) {
    const int64_t cw = int64_t(1) << sh;
    const int64_t per_block = div_up(div_up(W2, cw), std::max<int64_t>(n_blocks, 1));
    const int64_t trips = div_up(rows, (256 / cw) * 4);
    if (per_block * trips < best) {
      best = per_block * trips;
      best_shift = sh;
    }
  }
  return best_shift;
}

// force_S > 0: that many slabs per instance instead of the count the rules below arrive at.
inline ClPlan plan_cl_with(bool bwd, int V, int64_t N, int64_t C, int64_t D, int cus, int64_t force_S) {
  const Tuning& t = tuning();
  ClPlan p;
  p.V = V;
  p.CV = static_cast<int>(div_up(C, V));
  p.TPP = std::min(256, pow2_ceil(p.CV));
  const int tpp_full = p.TPP;
  const int max_u = bwd ? 8 : 16;
  bool single_pass = false;
  if (t.cl_fused && t.cl_fused_split && V > 1) {
    // Single pass: the D pixels of an instance, for a tile of TPP channel vectors, fit the
    // registers of one workgroup at max_u vectors per thread.  Narrower tiles (down to 8
    // vectors: 128-byte pieces of a pixel) hold more pixels each, and there are more of them:
    // the widest tile that fits is split further while the launch has fewer workgroups than CUs.
    int pick = 0;
    for (int tp = p.TPP; tp >= std::min(p.TPP, 8); tp >>= 1) {
      if (div_up(D, 256 / tp) > max_u) continue;
      if (pick == 0 || N * div_up(p.CV, pick) < cus) pick = tp;
    }
    if (pick != 0) {
      p.TPP = pick;
      single_pass = true;
    }
  }
  if (!single_pass && t.cl_narrow_tiles && V > 1 && C % (8 * V) == 0) {
    // Two stages: tiles of 8 channel vectors (128 bytes of a pixel) when a pixel is a whole
    // number of 128-byte lines, so that no line is shared between tiles (with C = 100 halves
    // both tiles of a pixel fetch most of its lines: twice the traffic, measured twice the
    // time).  More, narrower tiles need fewer slabs for the same number of workgroups (fewer
    // partials to fold) and leave no lane idle when C / V is not a power of two:
    // [8, 128, 64^3] 301 / 492 -> 268 / 465 us, [9, 512, 4096] 41.8 / 45.3 -> 27.8 / 35.5 us,
    // [1, 512, 1024] 21.8 / 13.1 -> 8.1 / 8.6 us.
    p.TPP = std::min(tpp_full, 8);
    while (div_up(p.CV, p.TPP) > 65535 && p.TPP < tpp_full) p.TPP *= 2;
  }
  while ((1 << p.tpp_shift) < p.TPP) ++p.tpp_shift;
  p.CT = static_cast<int>(div_up(p.CV, p.TPP));
  const int ppb = 256 / p.TPP;
  // The backward of a large tensor gets half as many slabs: every slab is a partial dgamma / dbeta
  // row for stage 2 to fold before it can start ([8, 64, 512^2] 248 -> 224 us, [2, 128^3, 32]
  // 229 -> 220 us, [32, 128, 128^2] 117 -> 106 us; below 2^25 elements the second workgroup per
  // CU is worth more: [64, 64, 4096] 29.1 against 30.2 us).
  const bool big = N * C * D >= (int64_t(1) << 25);
  const int items = bwd && big ? t.cl_bwd_big_items.load() : t.cl_items_per_cu.load();
  const int64_t want = div_up(int64_t(cus) * items, std::max<int64_t>(N * p.CT, 1));
  const int64_t max_s = std::max<int64_t>(1, D / (int64_t(ppb) * 4));
  // the kernels index the slab partials of an instance ([S][2][C] floats) with 32 bits
  const int64_t s_cap = std::min<int64_t>(4096, std::max<int64_t>(1, ((int64_t(1) << 31) - 1) / std::max<int64_t>(C, 1)));
  int64_t S = single_pass ? 1 : std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, max_s), s_cap));
  // the elements of a register-resident slab are addressed with 32-bit offsets from its first
  // pixel
  const bool slab32 = (int64_t(16) * ppb + 1) * C < (int64_t(1) << 32);
  // A stage-2 workgroup combines the S slab partials of its channels on fold_p lanes per
  // channel, and in one memory round trip while a lane has at most kPlanClFoldRegs of them.
  // Up to fold_above slabs it does so itself; beyond, a launch of its own does it once per
  // instance (128 when four lanes share a channel, i.e. tiles of 8 vectors:
  // [1, 64, 256^2] forward 15.9 -> 14.0 us without the extra launch).
  const int cap = p.TPP * V;
  const int fold_p = cap >= 256 ? 1 : std::min(64, 256 / cap);
  const int fold_above = fold_p >= 4 ? 2 * kClFoldAbove : kClFoldAbove;
  if (t.cl_fold_cap && slab32 && !single_pass) {
    // An instance small enough for register-resident slabs that stage 2 can fold by itself gets
    // no more slabs than that takes: its launches are bound by dependent round trips, and every
    // further slab is more partials for every stage-2 workgroup to read.  The count: a workgroup
    // per CU (a second wave of workgroups measured slower: [4, 64, 128^2] 10.7 / 13.0 us with 64
    // slabs against 13.2 / 14.7 us with 128, [3, 64, 20000] forward 12.2 against 14.3 us), but
    // at least as many as leave a thread 8 vectors (16 measured slower: [2, 64, 32768] forward
    // 12.0 against 13.0 us), else max_u.
    const int64_t one_per_cu = std::max<int64_t>(1, cus / std::max<int64_t>(N * p.CT, 1));
    const int64_t s_fold = std::min<int64_t>(int64_t(kPlanClFoldRegs) * fold_p, fold_above);
    for (const int u_lim : {8, max_u}) {
      const int64_t s_try = std::max(std::min(one_per_cu, s_fold), div_up(D, int64_t(ppb) * u_lim));
      if (s_try <= s_fold) {
        S = std::min(S, s_try);
        break;
      }
    }
  }
  if (force_S > 0 && !single_pass) S = std::min<int64_t>(force_S, std::min<int64_t>(max_s, s_cap));
  p.slab_len = round_up(div_up(D, S), ppb);
  p.S = static_cast<int>(div_up(D, p.slab_len));
  p.n_work = N * p.S * p.CT;
  p.grid = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(p.n_work, int64_t(cus) * 32)));
  // a slab of at most 16 (backward: 8, it holds x and dy) vectors per thread stays in
  // registers between its load and its use
  const int64_t per_thread = p.slab_len / ppb;
  for (int u = 4; slab32 && u <= max_u; u *= 2) {
    if (per_thread <= u) {
      p.U = u;
      break;
    }
  }
  const size_t sect = align256(sizeof(float) * size_t(N) * size_t(p.S) * size_t(C));
  // fwd: slab statistics [N*S][2][C] (mean, m2); bwd: part[N*S][2][C]; then the per-instance
  // merge of either, folded[N][2][C]
  p.off_a = 0;
  p.off_fold = 2 * sect;
  p.fold = p.S > fold_above && N <= 65535;
  // (the backward holds x and dy: 16 pixels per thread of both measured no better than two stages)
  if (t.cl_fused && slab32 && V > 1 && p.S == 1 && per_thread <= (bwd ? 8 : 16)) {
    p.fused = true;
    p.fused_u = std::max(1, pow2_ceil(per_thread));
  }
  p.ws_bytes = p.off_fold + align256(sizeof(float) * 2 * size_t(N) * size_t(C));
  const int cap_here = static_cast<int>(std::min<int64_t>(cap, C));
  // (slabs of at most 8 vectors per thread: with 16 the forward kernel does not fit the registers
  // of two workgroups per CU)
  const bool single_ok = t.cl_single && V > 1 && C % V == 0 && p.U > 0 && p.U <= 8 && !p.fold && !p.fused &&
                         p.S >= 2 && p.S <= kPlanClSingleMaxSlabs && cap <= kPlanClSingleMaxCap &&
                         div_up(cap_here, p.S) <= kPlanClSingleMaxOwned;
  p.single = single_ok && N % kPlanXcdCount == 0 && N <= 64 && p.n_work <= int64_t(cus) * 2;
  const int64_t xm_grid = round_up(N * p.CT, kPlanXcdCount) * p.S;
  p.single_xm = single_ok && !p.single && t.cl_single_xm && p.S <= cus / kPlanXcdCount * 2 &&
                xm_grid < (int64_t(1) << 31);
  if (p.single_xm) {
    p.single = true;
    p.xm_grid = static_cast<int>(xm_grid);
    p.xm_resident = div_up(N * p.CT, kPlanXcdCount) * p.S <= cus / kPlanXcdCount * 2;
    p.xm_fold = N > 1 && N <= 64 && p.xm_resident;
  }
  if (p.single) {
    // tagged pairs: 16 bytes per (instance, slab, channel); finals: 16 bytes per (instance, channel), twice
    p.off_tagged = 0;
    p.off_finals = align256(size_t(16) * size_t(N) * size_t(p.S) * size_t(C));
    p.off_finals_dev = p.off_finals + align256(size_t(16) * size_t(N) * size_t(C));
    p.off_claims = p.off_finals_dev + align256(size_t(16) * size_t(N) * size_t(C));
    p.ws_bytes = std::max(p.ws_bytes, p.off_claims + align256(size_t(4) * size_t(N) * size_t(p.CT) * size_t(p.S)));
    if (p.single_xm) {  // (the finals_dev section is not used; the per-instance sums take its place)
      p.off_xm_part = p.off_finals_dev;
    }
  }
  return p;
}

inline ClPlan plan_cl(bool bwd, int V, int64_t N, int64_t C, int64_t D, int cus) {
  const ClPlan p = plan_cl_with(bwd, V, N, C, D, cus, 0);
  const Tuning& t = tuning();
  if (p.single || p.fused || !t.cl_single || !t.cl_single_xm || V == 1) return p;
  // The slab count above suits the two-stage kernels (fewer, longer slabs when there are many
  // instances).  One launch and one pass over x (and dy) is worth more where it is possible:
  // with slabs of at most 8 vectors per thread, if an instance then has no more slabs than the
  // single-launch kernels take.  (A call that cannot use them, in place or under capture, runs
  // the two-stage kernels on these slabs.)
  const int ppb = 256 / p.TPP;
  const int64_t s_x = div_up(D, int64_t(ppb) * 8);
  if (s_x < 2 || s_x > kPlanClSingleMaxSlabs) return p;
  const ClPlan q = plan_cl_with(bwd, V, N, C, D, cus, s_x);
  return q.single ? q : p;
}

}  // namespace atexn
