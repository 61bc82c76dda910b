// Host-only check of the launch planner (atex_amd/csrc/plan.h) over a sweep of shapes: every
// plan must satisfy what the kernels and launchers assume of it.  Built and run by
// tests/test_plan_invariants.py with g++ (plan.h has no HIP dependency).  Exit status 0 and
// "ok <count>" on success; one line per violated invariant otherwise.
#include <cstdio>
#include <cstdlib>

#include "plan.h"

namespace atexn {
// the product library's planner: its parameters are constants
const Tuning& tuning() {
  static const Tuning t;
  return t;
}
}  // namespace atexn

using namespace atexn;

static long g_checked = 0, g_failed = 0;

#define EXPECT(cond, ...)                                   \
  do {                                                      \
    if (!(cond)) {                                          \
      ++g_failed;                                           \
      if (g_failed < 50) {                                  \
        std::printf("FAIL %s: ", #cond);                    \
        std::printf(__VA_ARGS__);                           \
        std::printf("\n");                                  \
      }                                                     \
    }                                                       \
  } while (0)

static void check_rows(RowsKind kind, bool layer_norm, int vec, int64_t n_rows, int64_t D, int C, int cus) {
  ++g_checked;
  const RowsRoute r = route_rows(kind, layer_norm, vec, n_rows, D);
  EXPECT(r.V == 1 || r.V == vec, "V=%d", r.V);
  EXPECT(r.V == 1 || D >= r.V, "vector path with D=%lld < V", (long long)D);
  const int64_t n_vec = div_up(D, r.V);
  if (r.small) {
    const SmallPlan p = plan_small(kind, r.V, n_rows, D, C, cus);
    EXPECT(p.NV >= 1 && p.NV <= kPlanSmallMaxVec, "NV=%d D=%lld", p.NV, (long long)D);
    EXPECT(p.grid >= 1 && int64_t(p.grid) <= int64_t(cus) * 8, "grid=%d", p.grid);
    if (kind == RowsKind::kBwdCols) {
      EXPECT(p.part_rows == p.grid && p.ws_bytes >= sizeof(float) * 2 * size_t(D) * size_t(p.grid), "small partial rows");
    }
    return;
  }
  if (r.tiles) {
    const bool bwd = kind != RowsKind::kFwd;
    const TilePlan p = plan_tiles(bwd, r.V, n_rows, D, cus);
    EXPECT(p.CW == int64_t(kPlanTileThreads) * kPlanTileVpt * r.V, "CW");
    EXPECT(int64_t(p.CT) * p.CW >= D && int64_t(p.CT - 1) * p.CW < D, "CT=%d D=%lld", p.CT, (long long)D);
    EXPECT(p.R >= 1 && int64_t(p.RS) * p.R >= n_rows && int64_t(p.RS - 1) * p.R < n_rows, "RS=%d R=%lld rows=%lld",
           p.RS, (long long)p.R, (long long)n_rows);
    EXPECT(p.RS <= 65535 && p.CT <= 65535, "grid dims RS=%d CT=%d", p.RS, p.CT);
    if (!bwd) {
      EXPECT(p.S >= 1 && int64_t(p.S) * p.chunk >= D && int64_t(p.S - 1) * p.chunk < D, "S=%d chunk=%lld", p.S, (long long)p.chunk);
      EXPECT(p.chunk % (256 * r.V) == 0, "chunk granularity");
      EXPECT(p.ws_bytes >= sizeof(float) * 2 * size_t(n_rows) * size_t(p.S), "stats workspace");
    } else {
      const int64_t cw = int64_t(kPlanTileThreads) * p.sums_vpt * r.V;
      EXPECT(int64_t(p.sums_CT) * cw >= D && int64_t(p.sums_CT - 1) * cw < D, "sums_CT");
      EXPECT(int64_t(p.sums_RS) * p.sums_R >= n_rows && int64_t(p.sums_RS - 1) * p.sums_R < n_rows, "sums_RS");
      EXPECT(p.off_rowsum >= sizeof(float) * 2 * size_t(n_rows) * size_t(p.sums_CT), "pairs section");
      EXPECT(p.off_part >= p.off_rowsum + sizeof(float) * 2 * size_t(n_rows), "rowsum section");
      EXPECT(p.ws_bytes >= p.off_part + (p.sums_RS > 1 ? sizeof(float) * 2 * size_t(D) * size_t(p.sums_RS) : 0), "part section");
    }
    return;
  }
  const RowsPlan p = plan_rows(kind, r.V, n_rows, D, layer_norm ? 0 : C, cus);
  EXPECT(p.ragged == (D % r.V != 0), "ragged");
  // the one-launch plan for channel-first planes, where a plan carries one (`before`: bytes of the
  // workspace sections that precede its tagged pairs)
  auto check_plane_single = [&](size_t before) {
  if (p.plane_single) {
    // what plane_fwd_single / plane_bwd_single assume: whole vectors, chunks of at most 8
    // vectors per thread of 512, no more chunks than lanes in a wave or than an XCD holds such
    // workgroups, a grid of whole planes per XCD, the tagged pairs behind the other sections
    const int64_t n_vec = D / r.V;
    EXPECT(D % r.V == 0 && r.V > 1 && C > 0, "plane single: D=%lld V=%d", (long long)D, r.V);
    EXPECT(p.ps_S >= 2 && p.ps_S <= 64 && p.ps_S <= cus / 8 * 2, "plane single: S=%d cus=%d", p.ps_S, cus);
    EXPECT(p.ps_chunk_vec >= 1 && p.ps_chunk_vec <= 512 * 8, "plane single: chunk of %d vectors", p.ps_chunk_vec);
    EXPECT(int64_t(p.ps_S - 1) * p.ps_chunk_vec < n_vec && n_vec <= int64_t(p.ps_S) * p.ps_chunk_vec,
           "plane single: S=%d chunk=%d n_vec=%lld", p.ps_S, p.ps_chunk_vec, (long long)n_vec);
    EXPECT(p.ps_full == (n_vec == int64_t(p.ps_S) * 4096), "plane single: full=%d", int(p.ps_full));
    EXPECT(int64_t(p.ps_grid) == (n_rows + 7) / 8 * 8 * p.ps_S, "plane single: grid=%d", p.ps_grid);
    EXPECT(p.off_ps_tagged % 256 == 0 && p.off_ps_tagged >= before &&
               p.ws_bytes >= p.off_ps_tagged + size_t(16) * size_t(n_rows) * size_t(p.ps_S),
           "plane single: workspace");
    if (kind == RowsKind::kBwdAffine) EXPECT(p.off_ps_tagged >= p.off_part + sizeof(float) * 2 * size_t(n_rows), "plane single: tagged pairs over the plane sums");
    EXPECT(p.off_ps_claims % 256 == 0 && p.off_ps_claims >= p.off_ps_tagged + size_t(16) * size_t(n_rows) * size_t(p.ps_S) &&
               p.ws_bytes >= p.off_ps_claims + size_t(4) * size_t(n_rows) * size_t(p.ps_S),
           "plane single: claim words");
    if (p.ps_fold) {
      EXPECT(kind == RowsKind::kBwdAffine && p.part_rows >= 1 && p.part_rows <= 64 && (C % 8 == 0 || p.part_rows == 1),
             "plane fold: N=%d C=%d", p.part_rows, C);
      EXPECT(p.off_ps_fold % 256 == 0 && p.off_ps_fold >= p.off_ps_claims + size_t(4) * size_t(n_rows) * size_t(p.ps_S) &&
                 p.ws_bytes >= p.off_ps_fold + size_t(16) * size_t(n_rows),
             "plane fold: workspace");
    }
  }
  };
  if (p.staged) {
    // the row staged in registers (8 vectors per thread) and LDS, 512 threads
    EXPECT(!p.resident && r.V > 1 && kind != RowsKind::kBwdCols && n_vec > resident_limit(kind), "staged with n_vec=%lld", (long long)n_vec);
    EXPECT(p.threads == 512 && p.nv_lds >= 1 && int64_t(8 + p.nv_lds) * 512 >= n_vec, "staged row not covered: nv_lds=%d n_vec=%lld", p.nv_lds, (long long)n_vec);
    EXPECT(p.fold_lds == size_t(p.nv_lds) * 512 * (kind == RowsKind::kFwd ? 16 : 32) && p.fold_lds + 512 <= 160 * 1024, "staged LDS bytes %zu", p.fold_lds);
    EXPECT(p.grid >= 1 && p.grid <= n_rows && int64_t(p.grid) * int64_t(p.fold_lds + 512) <= int64_t(cus) * 160 * 1024, "staged grid=%d", p.grid);
    if (kind == RowsKind::kBwdAffine) EXPECT(p.part_rows == n_rows / C && p.ws_bytes >= sizeof(float) * 2 * size_t(n_rows), "staged partial rows");
    check_plane_single(kind == RowsKind::kBwdAffine ? sizeof(float) * 2 * size_t(n_rows) : 0);
    return;
  }
  if (p.resident) {
    if (p.acc_lds) {
      // the LayerNorm backward with its column accumulators in LDS
      EXPECT(kind == RowsKind::kBwdCols && r.V > 1 && n_vec > resident_limit(kind) && n_vec <= 4096, "acc_lds with n_vec=%lld", (long long)n_vec);
      EXPECT(p.tpr == 0 && (p.vpt == 4 || p.vpt == 8) && !p.exact, "acc_lds launch shape");
      EXPECT(p.threads <= (p.vpt == 8 ? 512 : (r.V == 8 ? 640 : 1024)) && int64_t(p.threads) * p.vpt >= n_vec,
             "acc_lds threads=%d vpt=%d n_vec=%lld", p.threads, p.vpt, (long long)n_vec);
      EXPECT(p.fold_lds >= sizeof(float) * 2 * size_t(round_up(D, 4)) && p.fold_lds + 512 <= 160 * 1024, "acc_lds LDS bytes %zu", p.fold_lds);
      EXPECT(p.grid >= 1 && p.grid <= cus, "acc_lds grid=%d: one workgroup per CU", p.grid);
    } else {
      EXPECT(n_vec <= resident_limit(kind), "resident beyond the limit");
    }
    EXPECT(p.threads >= 64 && p.threads <= 1024 && p.threads % 64 == 0, "threads=%d", p.threads);
    EXPECT(p.vpt >= 1 && p.vpt <= 8, "vpt=%d", p.vpt);
    if (p.tpr == 0) {
      EXPECT(p.rpb == 1 && p.rb == 1, "block-per-row with rpb=%d rb=%d", p.rpb, p.rb);
      EXPECT(int64_t(p.threads) * p.vpt >= n_vec, "row not covered: threads=%d vpt=%d n_vec=%lld", p.threads, p.vpt,
             (long long)n_vec);
      // the launch bounds of the block-per-row kernels (768 threads with 2 vectors per thread, 512 otherwise)
      if (!p.acc_lds) EXPECT(p.threads <= (p.vpt == 2 ? 768 : (p.vpt == 4 && kind == RowsKind::kFwd ? 768 : 512)), "threads=%d vpt=%d exceed the kernel's launch bounds", p.threads, p.vpt);
    } else {
      EXPECT((p.tpr & (p.tpr - 1)) == 0 && p.tpr >= 8 && p.tpr <= 256, "tpr=%d", p.tpr);
      EXPECT(int64_t(p.tpr) * p.vpt >= n_vec, "row not covered: tpr=%d vpt=%d n_vec=%lld", p.tpr, p.vpt, (long long)n_vec);
      EXPECT(p.threads % p.tpr == 0 && p.rpb == p.threads / p.tpr, "rpb=%d threads=%d tpr=%d", p.rpb, p.threads, p.tpr);
      EXPECT(p.rb == 1 || p.tpr <= 64, "row batching with tpr=%d", p.tpr);
      EXPECT(p.rb == 1 || p.rb == 2 || p.rb == 4, "rb=%d", p.rb);
      if (p.tpr > 64) EXPECT(kind == RowsKind::kBwdCols && p.threads == 512, "wave groups outside the LN backward");
    }
    if (p.exact) {
      EXPECT(!p.ragged && r.V > 1, "exact but ragged / scalar");
      EXPECT(n_vec == int64_t(p.tpr == 0 ? p.threads : p.tpr) * p.vpt, "exact but lanes do not match the row");
      EXPECT(n_rows % (int64_t(p.rpb) * p.rb) == 0, "exact but rows do not fill the batches");
    }
    EXPECT(p.grid >= 1 && int64_t(p.grid) <= div_up(n_rows, int64_t(p.rpb) * p.rb), "grid=%d", p.grid);
    if (kind == RowsKind::kBwdCols) {
      EXPECT(p.part_rows == p.grid, "part_rows");
      EXPECT(p.ws_bytes >= sizeof(float) * 2 * size_t(D) * size_t(p.grid), "partial rows workspace");
      const int waves = p.threads / 64;
      if (p.tpr != 0) {
        EXPECT(waves <= kPlanFoldMaxWaves && waves % std::max(1, p.tpr / 64) == 0, "fold: %d waves, %d lanes per row", waves, p.tpr);
        const int w = r.V % 4 == 0 ? 4 : 1, lr = std::min(p.tpr, 64), q = 2 * r.V * p.vpt / w;
        const int per_pass = std::min(q, kPlanFoldLdsBytes / (kPlanFoldMaxWaves * lr * w * 4));
        EXPECT(per_pass >= 1 && (2 * r.V * p.vpt) % w == 0, "fold groups");
        EXPECT(p.fold_lds == size_t(waves) * per_pass * lr * w * sizeof(float), "fold_lds=%zu", p.fold_lds);
        EXPECT(p.fold_lds <= size_t(kPlanFoldLdsBytes), "fold_lds=%zu", p.fold_lds);
      }
    } else if (kind == RowsKind::kBwdAffine) {
      EXPECT(n_rows % C == 0 && p.part_rows == n_rows / C, "affine part rows");
      EXPECT(p.ws_bytes >= sizeof(float) * 2 * size_t(n_rows), "affine workspace");
      if (p.affine_fold) {
        // what the in-kernel fold over the batch assumes: q consecutive planes per workgroup and
        // step (1 with a workgroup per plane), a lane per instance, the planes of a channel group
        // handled on one XCD, its tagged pairs in the workspace
        const int64_t q = p.tpr == 0 ? 1 : int64_t(p.rpb) * p.rb;
        EXPECT((p.tpr == 0 ? p.rb == 1 : r.V > 1) && p.part_rows >= 2 && p.part_rows <= 64, "affine fold: tpr=%d N=%d", p.tpr, p.part_rows);
        EXPECT(C % q == 0 && (C / q) % 8 == 0 && p.grid % 8 == 0 && q <= 64 && p.part_rows * q <= 1024,
               "affine fold: C=%d q=%lld grid=%d", C, (long long)q, p.grid);
        EXPECT(p.off_tagged % 256 == 0 && p.off_tagged >= sizeof(float) * 2 * size_t(n_rows) &&
                   p.ws_bytes >= p.off_tagged + size_t(16) * size_t(n_rows),
               "affine fold: workspace");
        // channel group j (channels j * q ...) is folded by workgroup G-1 - (C/q-1-j) % G
        // (rows_bwd_resident): on the XCD of every workgroup that handles a plane of the group,
        // and started after all of them.  Step t of the row loop (planes t * q ...) runs on
        // workgroup t % G.
        const int64_t G = p.grid, cg = C / q;
        bool placed = true;
        for (int64_t j = 0; j < cg && placed; ++j) {
          const int64_t folder = G - 1 - (cg - 1 - j) % G;
          for (int64_t n = 0; n < p.part_rows; ++n) {
            const int64_t w = (n * cg + j) % G;
            if (w > folder || w % 8 != folder % 8) placed = false;
          }
        }
        EXPECT(placed, "affine fold: C=%d q=%lld grid=%d: a folding workgroup waits for a later one or another XCD's", C, (long long)q, p.grid);
      }
    }
  } else {
    EXPECT(!layer_norm, "LayerNorm rows beyond the resident limit go to the tiles");
    EXPECT(p.S >= 1 && int64_t(p.S) * p.chunk >= D && int64_t(p.S - 1) * p.chunk < D, "S=%d chunk=%lld D=%lld", p.S,
           (long long)p.chunk, (long long)D);
    EXPECT(p.chunk % (256 * r.V) == 0, "chunk granularity");
    EXPECT(p.split_grid >= 1 && int64_t(p.split_grid) <= n_rows * p.S, "split_grid");
    EXPECT(p.ws_bytes >= sizeof(float) * 2 * size_t(n_rows) * size_t(p.S), "pairs workspace");
    check_plane_single(sizeof(float) * 2 * size_t(n_rows) * size_t(p.S));
    if (kind == RowsKind::kBwdAffine) EXPECT(p.ws_bytes >= p.off_part + sizeof(float) * 2 * size_t(n_rows), "part workspace");
  }
}

static void check_cl(bool bwd, int V, int64_t N, int64_t C, int64_t D, int cus) {
  ++g_checked;
  const ClPlan p = plan_cl(bwd, V, N, C, D, cus);
  const int ppb = 256 / p.TPP;
  EXPECT(p.CV == div_up(C, V), "CV");
  EXPECT((p.TPP & (p.TPP - 1)) == 0 && p.TPP >= 1 && p.TPP <= 256 && (1 << p.tpp_shift) == p.TPP, "TPP=%d", p.TPP);
  EXPECT(int64_t(p.CT) * p.TPP >= p.CV, "CT=%d", p.CT);
  if (p.CT > 65535) return;  // more than 65535 tiles of 2048 channels: the launcher refuses the call
  EXPECT(p.S >= 1 && p.S <= 65535, "S=%d", p.S);
  EXPECT(p.slab_len >= 1 && int64_t(p.S) * p.slab_len >= D && int64_t(p.S - 1) * p.slab_len < D, "S=%d slab_len=%lld D=%lld",
         p.S, (long long)p.slab_len, (long long)D);
  // 32-bit positions inside the slab partials of an instance ([S][2][C] floats) ...
  EXPECT(2 * int64_t(p.S) * C < (int64_t(1) << 32), "partials of an instance beyond 32 bits: S=%d C=%lld", p.S, (long long)C);
  // ... and inside a register-resident slab
  if (p.U > 0 || p.fused) {
    const int u = p.fused ? p.fused_u : p.U;
    EXPECT(p.slab_len <= int64_t(u) * ppb, "slab of %lld pixels on %d slots x %d", (long long)p.slab_len, ppb, u);
    EXPECT((int64_t(u) * ppb + 1) * C < (int64_t(1) << 32), "resident slab beyond 32 bits: C=%lld", (long long)C);
    EXPECT(u <= (bwd ? 8 : 16), "u=%d", u);
  }
  if (p.fused) EXPECT(p.S == 1 && V > 1 && C >= V, "fused with S=%d", p.S);
  if (p.fold) EXPECT(p.S > kClFoldAbove && N <= 65535, "fold");
  EXPECT(p.n_work == N * p.S * p.CT && p.grid >= 1, "n_work");
  if (bwd) {
    // the chunk width of the dgamma / dbeta columns in stage 2: 64, 16, 4 or 1
    const int sh = cl_dparam_chunk_shift(p.fold ? N : N * p.S, 2 * C, p.n_work);
    EXPECT(sh == 0 || sh == 2 || sh == 4 || sh == 6, "chunk shift %d", sh);
  }
  const size_t sect = sizeof(float) * size_t(N) * size_t(p.S) * size_t(C);
  EXPECT(p.off_fold >= 2 * sect && p.ws_bytes >= p.off_fold + sizeof(float) * 2 * size_t(N) * size_t(C), "workspace sections");
  if (p.single) {
    // what cl_fwd_single / cl_bwd_single assume: resident slabs of at most 8 vectors, whole
    // channel vectors, a lane per slab and per instance, a tile's channels in LDS, every
    // workgroup on the chip at once, the workgroups of an instance on one XCD
    const int cap = p.TPP * V;
    EXPECT(V > 1 && C % V == 0 && p.U >= 4 && p.U <= 8 && !p.fused && !p.fold, "single: U=%d", p.U);
    EXPECT(p.S >= 2 && p.S <= 64, "single: S=%d", p.S);
    EXPECT(cap <= 64 && div_up(std::min<int64_t>(cap, C), p.S) <= 4, "single: cap=%d S=%d", cap, p.S);
    if (!p.single_xm) {
      // the (N, S, tiles) grid: every workgroup resident, an instance per XCD, a lane per instance
      EXPECT(N <= 64 && N % 8 == 0, "single: N=%lld", (long long)N);
      EXPECT(p.n_work <= int64_t(cus) * 2, "single: %lld workgroups on %d CUs", (long long)p.n_work, cus);
    } else {
      // the XCD-major grid: an instance's slabs fit one XCD, whole units per XCD, the
      // per-instance sums of the backward where the written-through finals would be
      EXPECT(p.S <= cus / 8 * 2, "single, XCD-major: S=%d on %d CUs", p.S, cus);
      EXPECT(int64_t(p.xm_grid) == (N * p.CT + 7) / 8 * 8 * p.S, "single, XCD-major: grid=%d", p.xm_grid);
      EXPECT(p.off_xm_part >= p.off_finals + size_t(16) * N * C && p.ws_bytes >= p.off_xm_part + sizeof(float) * 2 * N * C,
             "single, XCD-major: per-instance sums");
      if (p.xm_fold) {
        EXPECT(N > 1 && N <= 64 && (N * p.CT + 7) / 8 * p.S <= cus / 8 * 2, "single, XCD-major, fold in the kernel: N=%lld", (long long)N);
      }
    }
    EXPECT(p.off_tagged % 256 == 0 && p.off_finals >= p.off_tagged + size_t(16) * N * p.S * C &&
               p.off_finals_dev >= p.off_finals + size_t(16) * N * C &&
               p.off_claims % 256 == 0 && p.off_claims >= p.off_finals_dev + size_t(16) * N * C &&
               p.ws_bytes >= p.off_claims + size_t(4) * N * p.CT * p.S,
           "single: workspace sections");
  }
}

int main() {
  const int cus_list[] = {256, 304, 64, 1};
  const int64_t rows_list[] = {1, 2, 7, 32, 255, 256, 1000, 4096, 8192, 100000, 262144, 10000000};
  for (int cus : cus_list) {
    for (int vec : {4, 8}) {
      for (int64_t n_rows : rows_list) {
        for (int64_t D = 1; D <= 300000; D += (D < 4200 ? 1 : (D < 40000 ? 97 : 4099))) {
          check_rows(RowsKind::kFwd, true, vec, n_rows, D, 1, cus);
          check_rows(RowsKind::kBwdCols, true, vec, n_rows, D, 1, cus);
        }
      }
      // channel-first InstanceNorm: rows = N * C planes
      for (int64_t N : {1, 2, 8, 64, 100}) {
        for (int C : {1, 3, 32, 64, 100, 1024}) {
          for (int64_t D = 1; D <= 3000000; D += (D < 2100 ? 1 : (D < 70000 ? 211 : 65537))) {
            check_rows(RowsKind::kFwd, false, vec, N * C, D, C, cus);
            check_rows(RowsKind::kBwdAffine, false, vec, N * C, D, C, cus);
          }
        }
      }
      // channels-last InstanceNorm
      for (int64_t N : {1, 2, 8, 16, 64, 100, 16384, 70000}) {
        for (int64_t C : {1, 3, 8, 16, 32, 64, 100, 256, 520, 2048, 4096, 100000, 1048576, 3000000, 600000000}) {
          for (int64_t D : {1, 2, 5, 32, 64, 100, 1000, 4096, 16384, 262144, 2097152, 16777216}) {
            if (double(N) * double(C) * double(D) > 4e12) continue;
            const int V = C >= vec ? vec : 1;
            check_cl(false, V, N, C, D, cus);
            check_cl(true, V, N, C, D, cus);
          }
        }
      }
    }
  }
  if (g_failed) {
    std::printf("%ld of %ld plans violate an invariant\n", g_failed, g_checked);
    return 1;
  }
  std::printf("ok %ld\n", g_checked);
  return 0;
}
