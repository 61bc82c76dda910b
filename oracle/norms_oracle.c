/*
 * CPU ORACLE for the fused LayerNorm / InstanceNorm forward and backward ops.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against and the CPU baseline that the benchmark times; the shipped
 * library never links, loads or calls it.
 *
 * It restates, in plain C loops, the algorithm of the reference's CPU functors:
 *   LayerNorm forward      atex/nv_norms/cc/kernels/fused_layer_norm_op.cc:27-85
 *   LayerNorm backward     atex/nv_norms/cc/kernels/fused_layer_norm_op.cc:87-223
 *   InstanceNorm forward   atex/nv_norms/cc/kernels/fused_instance_norm_op.cc:39-108
 *   InstanceNorm backward  atex/nv_norms/cc/kernels/fused_instance_norm_op.cc:110-284
 * (mean -> centred sum of squares -> rsqrt(var + eps) -> scale/shift; backward as
 *  dl_dx + dl_dvar * dvar_dx + dl_dmean * dmean_dx with the same intermediate terms).
 *
 * Two arithmetic flavours of every function:
 *   *_f32  accumulates in float like the reference functor (U = float) and writes
 *          outputs in the op's own types (y/dx in the storage type, stats fp32);
 *          it is also what the benchmark times as the CPU baseline (OpenMP over
 *          rows / instances).
 *   *_f64  runs the identical formulae in double and writes UNROUNDED double
 *          outputs; the parity tests use it as the ground truth so that the
 *          summation order of either side does not enter the comparison.
 *
 * Pinning (see tests/test_oracle_*.py): both flavours are checked against torch's
 * CPU float64 native_layer_norm / group_norm and autograd, against a re-derivation
 * of the numpy closed forms in the reference's own tests
 * (tests/fused_layer_norm_test.py:20-62, tests/fused_instance_norm_test.py:21-65),
 * against finite differences and against row invariants.  What is NOT pinned: the
 * last-ulp fp16 rounding behaviour of tf.keras / tensorflow_addons (neither library
 * is available), which sits far inside the stated fp16 tolerance.
 *
 * Storage types: 0 = float32, 1 = float16 (IEEE binary16), 2 = bfloat16.
 * Layouts for InstanceNorm: channel_first != 0 -> x is [N, C, D]; else [N, D, C].
 * Saved statistics are mean and INVERSE STANDARD DEVIATION rsqrt(var + eps), with
 * the biased variance, as in the reference (norm_util.h:253-258).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { ORACLE_F32 = 0, ORACLE_F16 = 1, ORACLE_BF16 = 2 };

/* ---------------------------------------------------------------- conversions */

static inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

static inline float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_to_float(sign);
    /* subnormal: value = man * 2^-24 */
    float v = (float)man * 5.9604644775390625e-8f;
    return sign ? -v : v;
  }
  if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
  return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even float -> binary16 */
static inline uint16_t float_to_half(float f) {
  uint32_t x = float_to_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  }
  if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x38800000u) { /* subnormal half or zero */
    if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
    uint32_t e = ax >> 23;
    uint32_t m = (ax & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e; /* 14..24 */
    uint32_t r = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
  }
  uint32_t r = ax - 0x38000000u; /* rebias */
  uint32_t rem = r & 0x1fffu;
  r >>= 13;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
  return (uint16_t)(sign | r);
}

static inline float bf16_to_float(uint16_t b) { return bits_to_float((uint32_t)b << 16); }

static inline uint16_t float_to_bf16(float f) {
  uint32_t x = float_to_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

static inline double load_elem(int dtype, const void* p, size_t i) {
  switch (dtype) {
    case ORACLE_F32: return (double)((const float*)p)[i];
    case ORACLE_F16: return (double)half_to_float(((const uint16_t*)p)[i]);
    default: return (double)bf16_to_float(((const uint16_t*)p)[i]);
  }
}
static inline float load_elem_f(int dtype, const void* p, size_t i) {
  switch (dtype) {
    case ORACLE_F32: return ((const float*)p)[i];
    case ORACLE_F16: return half_to_float(((const uint16_t*)p)[i]);
    default: return bf16_to_float(((const uint16_t*)p)[i]);
  }
}
static inline void store_elem_f(int dtype, void* p, size_t i, float v) {
  switch (dtype) {
    case ORACLE_F32: ((float*)p)[i] = v; break;
    case ORACLE_F16: ((uint16_t*)p)[i] = float_to_half(v); break;
    default: ((uint16_t*)p)[i] = float_to_bf16(v); break;
  }
}

/* Exposed so the tests can pin the conversions against numpy / torch. */
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t oracle_float_to_half(float f) { return float_to_half(f); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
uint16_t oracle_float_to_bf16(float f) { return float_to_bf16(f); }

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
void oracle_set_num_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* Strided element access: element j of a "row" lives at base + j * stride.
 * LayerNorm and channel-first InstanceNorm rows have stride 1; a channels-last
 * (n, c) instance has base n*D*C + c and stride C
 * (fused_instance_norm_op.cc:47-52 picks the reduced dimension the same way). */

/* ------------------------------------------------------------------ forward */

#define DEFINE_ROW_FWD(NAME, ACC, LOAD, RSQRT)                                           \
  static void NAME(int dtype, const void* x, size_t base, size_t stride, size_t D,   \
                   ACC eps, ACC* mean_out, ACC* rstd_out) {                          \
    ACC d_inv = (ACC)1 / (ACC)D;                                                     \
    ACC s = 0;                                                                       \
    for (size_t j = 0; j < D; ++j) s += (ACC)LOAD(dtype, x, base + j * stride);      \
    ACC mean = s * d_inv;                                                            \
    ACC q = 0;                                                                       \
    for (size_t j = 0; j < D; ++j) {                                                 \
      ACC c = (ACC)LOAD(dtype, x, base + j * stride) - mean;                         \
      q += c * c;                                                                    \
    }                                                                                \
    *mean_out = mean;                                                                \
    *rstd_out = RSQRT(q * d_inv + eps);                                              \
  }

/* The float flavour rounds the square root and the divide in float, like the
 * functor's Eigen rsqrt on a float tensor. */
static inline float rsqrt_f32(float v) { return 1.0f / sqrtf(v); }
static inline double rsqrt_f64(double v) { return 1.0 / sqrt(v); }

DEFINE_ROW_FWD(row_stats_f32, float, load_elem_f, rsqrt_f32)
DEFINE_ROW_FWD(row_stats_f64, double, load_elem, rsqrt_f64)

void oracle_ln_fwd_f32(int dtype, const void* x, const float* gamma, const float* beta,
                       int64_t N, int64_t D, float eps, void* y, float* mean,
                       float* inv_std) {
  if (N <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    size_t base = (size_t)i * (size_t)D;
    float m, r;
    row_stats_f32(dtype, x, base, 1, (size_t)D, eps, &m, &r);
    for (int64_t j = 0; j < D; ++j) {
      float c = load_elem_f(dtype, x, base + j) - m;
      store_elem_f(dtype, y, base + j, c * (r * gamma[j]) + beta[j]);
    }
    mean[i] = m;
    inv_std[i] = r;
  }
}

void oracle_ln_fwd_f64(int dtype, const void* x, const float* gamma, const float* beta,
                       int64_t N, int64_t D, double eps, double* y, double* mean,
                       double* inv_std) {
  if (N <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    size_t base = (size_t)i * (size_t)D;
    double m, r;
    row_stats_f64(dtype, x, base, 1, (size_t)D, eps, &m, &r);
    for (int64_t j = 0; j < D; ++j) {
      double c = load_elem(dtype, x, base + j) - m;
      y[base + j] = c * (r * (double)gamma[j]) + (double)beta[j];
    }
    mean[i] = m;
    inv_std[i] = r;
  }
}

/* ----------------------------------------------------------------- backward */
/* Per row, with xc = x - mean, r = inv_std, g = dy * gamma   (LN.cc:177-221):
 *   dl_dx    = g * r
 *   dl_dvar  = sum_j dl_dx * xc * (-0.5) * r * r
 *   dvar_dx  = 2 * xc / D
 *   dl_dmean = sum_j (-dl_dx)  +  sum_j dl_dvar * (-2 / D) * xc
 *   dx       = dl_dx + dl_dvar * dvar_dx + dl_dmean / D
 * and over rows:  dgamma_j = sum_i dy * xc * r ,  dbeta_j = sum_i dy.
 * The mean and inv_std are INPUTS (the saved forward statistics), not recomputed. */

#define DEFINE_ROW_BWD(NAME, ACC, LOAD)                                                 \
  static void NAME(int dtype, const void* dy, const void* x, size_t base, size_t stride, \
                   size_t D, const float* gamma, size_t gamma_stride, ACC mean, ACC r,  \
                   ACC* dl_dvar_out, ACC* dl_dmean_out) {                               \
    ACC d_inv = (ACC)1 / (ACC)D;                                                        \
    ACC dl_dvar = 0, neg_sum = 0, xc_sum = 0;                                           \
    for (size_t j = 0; j < D; ++j) {                                                    \
      ACC xc = (ACC)LOAD(dtype, x, base + j * stride) - mean;                           \
      ACC dl_dx = (ACC)LOAD(dtype, dy, base + j * stride) *                             \
                  (ACC)gamma[j * gamma_stride] * r;                                     \
      dl_dvar += dl_dx * xc * (ACC)(-0.5) * r * r;                                      \
      neg_sum += -dl_dx;                                                                \
      xc_sum += xc;                                                                     \
    }                                                                                   \
    *dl_dvar_out = dl_dvar;                                                             \
    *dl_dmean_out = neg_sum + dl_dvar * (ACC)(-2) * d_inv * xc_sum;                     \
  }

DEFINE_ROW_BWD(row_bwd_f32, float, load_elem_f)
DEFINE_ROW_BWD(row_bwd_f64, double, load_elem)

void oracle_ln_bwd_f32(int dtype, const void* dy, const void* x, const float* gamma,
                       const float* mean, const float* inv_std, int64_t N, int64_t D,
                       void* dx, float* dgamma, float* dbeta) {
  if (D > 0) {
    memset(dgamma, 0, sizeof(float) * (size_t)D);
    memset(dbeta, 0, sizeof(float) * (size_t)D);
  }
  if (N <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    size_t base = (size_t)i * (size_t)D;
    float m = mean[i], r = inv_std[i], dl_dvar, dl_dmean;
    row_bwd_f32(dtype, dy, x, base, 1, (size_t)D, gamma, 1, m, r, &dl_dvar, &dl_dmean);
    float d_inv = 1.0f / (float)D;
    for (int64_t j = 0; j < D; ++j) {
      float xc = load_elem_f(dtype, x, base + j) - m;
      float dl_dx = load_elem_f(dtype, dy, base + j) * gamma[j] * r;
      store_elem_f(dtype, dx, base + j,
                   dl_dx + dl_dvar * (2.0f * xc * d_inv) + dl_dmean * d_inv);
    }
  }
  /* column sums over rows; blocked over columns so threads own disjoint outputs */
  const int64_t CB = 256;
#pragma omp parallel for schedule(static)
  for (int64_t j0 = 0; j0 < D; j0 += CB) {
    int64_t j1 = j0 + CB < D ? j0 + CB : D;
    for (int64_t i = 0; i < N; ++i) {
      size_t base = (size_t)i * (size_t)D;
      float m = mean[i], r = inv_std[i];
      for (int64_t j = j0; j < j1; ++j) {
        float dyv = load_elem_f(dtype, dy, base + j);
        float xs = (load_elem_f(dtype, x, base + j) - m) * r;
        dgamma[j] += dyv * xs;
        dbeta[j] += dyv;
      }
    }
  }
}

void oracle_ln_bwd_f64(int dtype, const void* dy, const void* x, const float* gamma,
                       const double* mean, const double* inv_std, int64_t N, int64_t D,
                       double* dx, double* dgamma, double* dbeta) {
  for (int64_t j = 0; j < D; ++j) dgamma[j] = dbeta[j] = 0.0;
  if (N <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N; ++i) {
    size_t base = (size_t)i * (size_t)D;
    double m = mean[i], r = inv_std[i], dl_dvar, dl_dmean;
    row_bwd_f64(dtype, dy, x, base, 1, (size_t)D, gamma, 1, m, r, &dl_dvar, &dl_dmean);
    double d_inv = 1.0 / (double)D;
    for (int64_t j = 0; j < D; ++j) {
      double xc = load_elem(dtype, x, base + j) - m;
      double dl_dx = load_elem(dtype, dy, base + j) * (double)gamma[j] * r;
      dx[base + j] = dl_dx + dl_dvar * (2.0 * xc * d_inv) + dl_dmean * d_inv;
    }
  }
  for (int64_t i = 0; i < N; ++i) {
    size_t base = (size_t)i * (size_t)D;
    double m = mean[i], r = inv_std[i];
    for (int64_t j = 0; j < D; ++j) {
      double dyv = load_elem(dtype, dy, base + j);
      dgamma[j] += dyv * (load_elem(dtype, x, base + j) - m) * r;
      dbeta[j] += dyv;
    }
  }
}

/* ------------------------------------------------------------ instance norm */

static inline void in_addr(int channel_first, int64_t n, int64_t c, int64_t C, int64_t D,
                           size_t* base, size_t* stride) {
  if (channel_first) {
    *base = ((size_t)n * (size_t)C + (size_t)c) * (size_t)D;
    *stride = 1;
  } else {
    *base = (size_t)n * (size_t)D * (size_t)C + (size_t)c;
    *stride = (size_t)C;
  }
}

void oracle_in_fwd_f32(int dtype, int channel_first, const void* x, const float* gamma,
                       const float* beta, int64_t N, int64_t C, int64_t D, float eps,
                       void* y, float* mean, float* inv_std) {
  if (N <= 0 || C <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t nc = 0; nc < N * C; ++nc) {
    int64_t n = nc / C, c = nc % C;
    size_t base, stride;
    in_addr(channel_first, n, c, C, D, &base, &stride);
    float m, r;
    row_stats_f32(dtype, x, base, stride, (size_t)D, eps, &m, &r);
    float sc = r * gamma[c], of = beta[c];
    for (int64_t j = 0; j < D; ++j) {
      size_t a = base + (size_t)j * stride;
      store_elem_f(dtype, y, a, (load_elem_f(dtype, x, a) - m) * sc + of);
    }
    mean[nc] = m;
    inv_std[nc] = r;
  }
}

void oracle_in_fwd_f64(int dtype, int channel_first, const void* x, const float* gamma,
                       const float* beta, int64_t N, int64_t C, int64_t D, double eps,
                       double* y, double* mean, double* inv_std) {
  if (N <= 0 || C <= 0 || D <= 0) return;
#pragma omp parallel for schedule(static)
  for (int64_t nc = 0; nc < N * C; ++nc) {
    int64_t n = nc / C, c = nc % C;
    size_t base, stride;
    in_addr(channel_first, n, c, C, D, &base, &stride);
    double m, r;
    row_stats_f64(dtype, x, base, stride, (size_t)D, eps, &m, &r);
    double sc = r * (double)gamma[c], of = (double)beta[c];
    for (int64_t j = 0; j < D; ++j) {
      size_t a = base + (size_t)j * stride;
      y[a] = (load_elem(dtype, x, a) - m) * sc + of;
    }
    mean[nc] = m;
    inv_std[nc] = r;
  }
}

/* Backward (IN.cc:232-281): the LayerNorm row formulae applied to every (n, c)
 * instance with the channel's scalar gamma, then dgamma_c / dbeta_c summed over the
 * batch and the spatial positions. */
void oracle_in_bwd_f32(int dtype, int channel_first, const void* dy, const void* x,
                       const float* gamma, const float* mean, const float* inv_std,
                       int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
                       float* dbeta) {
  for (int64_t c = 0; c < C; ++c) dgamma[c] = dbeta[c] = 0.f;
  if (N <= 0 || C <= 0 || D <= 0) return;
  float* dg_nc = (float*)malloc(sizeof(float) * (size_t)(N * C));
  float* db_nc = (float*)malloc(sizeof(float) * (size_t)(N * C));
#pragma omp parallel for schedule(static)
  for (int64_t nc = 0; nc < N * C; ++nc) {
    int64_t n = nc / C, c = nc % C;
    size_t base, stride;
    in_addr(channel_first, n, c, C, D, &base, &stride);
    float m = mean[nc], r = inv_std[nc], dl_dvar, dl_dmean;
    row_bwd_f32(dtype, dy, x, base, stride, (size_t)D, gamma + c, 0, m, r, &dl_dvar,
                &dl_dmean);
    float d_inv = 1.0f / (float)D, dg = 0.f, db = 0.f, gc = gamma[c];
    for (int64_t j = 0; j < D; ++j) {
      size_t a = base + (size_t)j * stride;
      float xc = load_elem_f(dtype, x, a) - m;
      float dyv = load_elem_f(dtype, dy, a);
      float dl_dx = dyv * gc * r;
      store_elem_f(dtype, dx, a, dl_dx + dl_dvar * (2.0f * xc * d_inv) + dl_dmean * d_inv);
      dg += dyv * (xc * r);
      db += dyv;
    }
    dg_nc[nc] = dg;
    db_nc[nc] = db;
  }
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c) {
      dgamma[c] += dg_nc[n * C + c];
      dbeta[c] += db_nc[n * C + c];
    }
  free(dg_nc);
  free(db_nc);
}

void oracle_in_bwd_f64(int dtype, int channel_first, const void* dy, const void* x,
                       const float* gamma, const double* mean, const double* inv_std,
                       int64_t N, int64_t C, int64_t D, double* dx, double* dgamma,
                       double* dbeta) {
  for (int64_t c = 0; c < C; ++c) dgamma[c] = dbeta[c] = 0.0;
  if (N <= 0 || C <= 0 || D <= 0) return;
  double* dg_nc = (double*)malloc(sizeof(double) * (size_t)(N * C));
  double* db_nc = (double*)malloc(sizeof(double) * (size_t)(N * C));
#pragma omp parallel for schedule(static)
  for (int64_t nc = 0; nc < N * C; ++nc) {
    int64_t n = nc / C, c = nc % C;
    size_t base, stride;
    in_addr(channel_first, n, c, C, D, &base, &stride);
    double m = mean[nc], r = inv_std[nc], dl_dvar, dl_dmean;
    row_bwd_f64(dtype, dy, x, base, stride, (size_t)D, gamma + c, 0, m, r, &dl_dvar,
                &dl_dmean);
    double d_inv = 1.0 / (double)D, dg = 0.0, db = 0.0, gc = (double)gamma[c];
    for (int64_t j = 0; j < D; ++j) {
      size_t a = base + (size_t)j * stride;
      double xc = load_elem(dtype, x, a) - m;
      double dyv = load_elem(dtype, dy, a);
      dx[a] = dyv * gc * r + dl_dvar * (2.0 * xc * d_inv) + dl_dmean * d_inv;
      dg += dyv * (xc * r);
      db += dyv;
    }
    dg_nc[nc] = dg;
    db_nc[nc] = db;
  }
  for (int64_t n = 0; n < N; ++n)
    for (int64_t c = 0; c < C; ++c) {
      dgamma[c] += dg_nc[n * C + c];
      dbeta[c] += db_nc[n * C + c];
    }
  free(dg_nc);
  free(db_nc);
}
