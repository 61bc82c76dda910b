// Host (CPU) kernels behind the same four ops: what runs when the op's tensors live in host
// memory.  The reference registers CPU kernels next to its GPU ones
// (fused_layer_norm_op.cc:465-478, fused_instance_norm_op.cc:541-554; functors
// fused_layer_norm_op.cc:27-223, fused_instance_norm_op.cc:39-284, built from Eigen tensor
// expressions); these are their counterpart, written as plain loops:
//
//   forward   mean = sum(x) / D;  inv_std = rsqrt(sum((x - mean)^2) / D + eps)   (two passes
//             over the row, like the functor's x.sum() and x_centered.square().sum());
//             y = (x - mean) * inv_std * gamma + beta
//   backward  dgamma = sum dy * (x - mean) * inv_std, dbeta = sum dy,
//             dx = inv_std * (g - (s1 + xh * s2) / D),  g = dy * gamma, xh = (x - mean) * inv_std,
//             s1 = sum g, s2 = sum g * xh: the functor's dl_dx + dl_dvar * 2 (x - mean) / D +
//             dl_dmean / D with dl_dvar = -1/2 inv_std^3 sum g (x - mean) and
//             dl_dmean = -inv_std s1 (its extra dl_dvar * (-2 / D) * sum(x - mean) term is zero)
//
// Storage T in {float, half, bfloat16} is converted to float once per element; element-wise
// arithmetic is float, sums are carried in double (a row can hold 10^7 elements), statistics
// and parameter gradients are stored as float.  Work is split over host threads by rows /
// planes / instances; dgamma / dbeta are summed in an order that does not depend on the
// number of threads, so results are reproducible run to run and machine to machine.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "cpu_kernels.h"

namespace atexn {
namespace cpu {
namespace {

// ----------------------------------------------------------------- storage conversions
inline float load_as_float(const float* p, int64_t i) { return p[i]; }
inline void store_from_float(float* p, int64_t i, float v) { p[i] = v; }

struct Half {
  uint16_t bits;
};
struct BFloat16 {
  uint16_t bits;
};

inline float bits_to_float(uint32_t u) {
  float f;
  std::memcpy(&f, &u, 4);
  return f;
}
inline uint32_t float_to_bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

// IEEE binary16 -> binary32, exact (subnormals via one float multiply).
inline float load_as_float(const Half* p, int64_t i) {
  const uint32_t h = p[i].bits;
  const uint32_t sign = (h & 0x8000u) << 16;
  const uint32_t em = h & 0x7FFFu;
  if (em >= 0x7C00u) return bits_to_float(sign | 0x7F800000u | ((em & 0x3FFu) << 13));  // inf / nan
  if (em < 0x0400u) {                                                                   // zero / subnormal
    const float mag = static_cast<float>(em) * 5.9604644775390625e-8f;                  // em * 2^-24
    return bits_to_float(sign | float_to_bits(mag));
  }
  return bits_to_float(sign | ((em + (112u << 10)) << 13));
}
// binary32 -> binary16, round to nearest even.
inline void store_from_float(Half* p, int64_t i, float v) {
  const uint32_t u = float_to_bits(v);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const uint32_t a = u & 0x7FFFFFFFu;
  uint16_t out;
  if (a >= 0x7F800000u) {
    out = static_cast<uint16_t>(sign | 0x7C00u | (a > 0x7F800000u ? 0x200u | ((a >> 13) & 0x3FFu) : 0u));
  } else if (a >= 0x477FF000u) {  // rounds to 65520 or more: infinity
    out = static_cast<uint16_t>(sign | 0x7C00u);
  } else if (a < 0x38800000u) {   // below the smallest normal half: subnormal or zero
    if (a < 0x33000000u) {        // below half of the smallest subnormal
      out = static_cast<uint16_t>(sign);
    } else {
      const int e = static_cast<int>(a >> 23);                  // biased float exponent, 102 .. 112
      const uint32_t m = (a & 0x7FFFFFu) | 0x800000u;           // 24-bit significand
      const int shift = 126 - e;                                // 14 .. 24
      uint32_t q = m >> shift;
      const uint32_t rem = m & ((1u << shift) - 1u);
      const uint32_t halfway = 1u << (shift - 1);
      if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
      out = static_cast<uint16_t>(sign | q);
    }
  } else {
    const uint32_t r = a + 0xFFFu + ((a >> 13) & 1u);           // round to nearest even at bit 13
    out = static_cast<uint16_t>(sign | ((r - (112u << 23)) >> 13));
  }
  p[i].bits = out;
}

inline float load_as_float(const BFloat16* p, int64_t i) {
  return bits_to_float(static_cast<uint32_t>(p[i].bits) << 16);
}
inline void store_from_float(BFloat16* p, int64_t i, float v) {
  const uint32_t u = float_to_bits(v);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) {  // nan: keep it a nan
    p[i].bits = static_cast<uint16_t>((u >> 16) | 0x40u);
    return;
  }
  p[i].bits = static_cast<uint16_t>((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// ------------------------------------------------------------------------ threading
int thread_limit() {
  static const int limit = [] {
    int n = static_cast<int>(std::thread::hardware_concurrency());
    if (const char* env = std::getenv("ATEXN_CPU_THREADS")) n = std::atoi(env);
    return std::max(1, std::min(n, 64));
  }();
  return limit;
}

// fn(begin, end) over [0, n) cut into contiguous ranges, one per thread; small jobs run inline.
template <typename Fn>
void parallel_ranges(int64_t n, int64_t min_items_per_thread, Fn fn) {
  if (n <= 0) return;
  const int64_t want = std::max<int64_t>(1, n / std::max<int64_t>(1, min_items_per_thread));
  const int threads = static_cast<int>(std::min<int64_t>(thread_limit(), want));
  if (threads <= 1) {
    fn(int64_t(0), n);
    return;
  }
  std::vector<std::thread> pool;
  pool.reserve(threads - 1);
  const int64_t per = (n + threads - 1) / threads;
  for (int t = 1; t < threads; ++t) {
    const int64_t b = t * per, e = std::min<int64_t>(n, b + per);
    if (b < e) pool.emplace_back([=] { fn(b, e); });
  }
  fn(int64_t(0), std::min<int64_t>(n, per));
  for (auto& th : pool) th.join();
}

// Rows of a thread are worth spreading once a job has this many elements per thread.
constexpr int64_t kMinElemsPerThread = 1 << 15;

inline int64_t rows_per_thread_floor(int64_t row_len) {
  return std::max<int64_t>(1, kMinElemsPerThread / std::max<int64_t>(1, row_len));
}

// ------------------------------------------------------------- contiguous rows
// Statistics of one contiguous row (two passes).
template <typename T>
inline void row_stats(const T* x, int64_t D, float eps, float* mean_out, float* rstd_out) {
  double s = 0.0;
  for (int64_t j = 0; j < D; ++j) s += load_as_float(x, j);
  const float mean = static_cast<float>(s / static_cast<double>(D));
  double q = 0.0;
  for (int64_t j = 0; j < D; ++j) {
    const float d = load_as_float(x, j) - mean;
    q += static_cast<double>(d) * d;
  }
  *mean_out = mean;
  *rstd_out = static_cast<float>(1.0 / std::sqrt(q / static_cast<double>(D) + static_cast<double>(eps)));
}

// The two row sums of the backward: s1 = sum g, s2 = sum g * xh, g = dy * gamma_j (LayerNorm:
// gamma per column) or dy * gamma_c (InstanceNorm: `gamma` is null and `scalar_gamma` is used).
template <typename T>
inline void row_bwd_sums(const T* dy, const T* x, const float* gamma, float scalar_gamma, float mean,
                         float rstd, int64_t D, double* s1_out, double* s2_out) {
  double s1 = 0.0, s2 = 0.0;
  for (int64_t j = 0; j < D; ++j) {
    const float g = load_as_float(dy, j) * (gamma ? gamma[j] : scalar_gamma);
    const float xh = (load_as_float(x, j) - mean) * rstd;
    s1 += g;
    s2 += static_cast<double>(g) * xh;
  }
  *s1_out = s1;
  *s2_out = s2;
}

template <typename T>
inline void row_bwd_dx(const T* dy, const T* x, const float* gamma, float scalar_gamma, float mean,
                       float rstd, int64_t D, double s1, double s2, T* dx) {
  const float inv_d = 1.0f / static_cast<float>(D);
  const float a = static_cast<float>(s1) * inv_d, b = static_cast<float>(s2) * inv_d;
  for (int64_t j = 0; j < D; ++j) {
    const float g = load_as_float(dy, j) * (gamma ? gamma[j] : scalar_gamma);
    const float xh = (load_as_float(x, j) - mean) * rstd;
    store_from_float(dx, j, rstd * (g - (a + xh * b)));
  }
}

template <typename T>
void layer_norm_fwd_t(const T* x, const float* gamma, const float* beta, int64_t N, int64_t D,
                      float eps, T* y, float* mean, float* rstd) {
  parallel_ranges(N, rows_per_thread_floor(D), [=](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r) {
      const T* xr = x + r * D;
      T* yr = y + r * D;
      float m, s;
      row_stats(xr, D, eps, &m, &s);
      for (int64_t j = 0; j < D; ++j) {
        store_from_float(yr, j, (load_as_float(xr, j) - m) * s * gamma[j] + beta[j]);
      }
      mean[r] = m;
      rstd[r] = s;
    }
  });
}

// Rows are cut into at most kColumnSumBlocks contiguous blocks, whatever the thread count; a
// block's column sums are accumulated row by row and the blocks are then added in order, so
// dgamma / dbeta do not depend on how many threads ran.
constexpr int64_t kColumnSumBlocks = 32;

template <typename T>
void layer_norm_bwd_t(const T* dy, const T* x, const float* gamma, const float* mean,
                      const float* rstd, int64_t N, int64_t D, T* dx, float* dgamma, float* dbeta) {
  // dx: rows are independent
  parallel_ranges(N, rows_per_thread_floor(D), [=](int64_t r0, int64_t r1) {
    for (int64_t r = r0; r < r1; ++r) {
      double s1, s2;
      row_bwd_sums(dy + r * D, x + r * D, gamma, 0.f, mean[r], rstd[r], D, &s1, &s2);
      row_bwd_dx(dy + r * D, x + r * D, gamma, 0.f, mean[r], rstd[r], D, s1, s2, dx + r * D);
    }
  });
  // dgamma / dbeta
  if (D >= 64 * static_cast<int64_t>(thread_limit())) {
    // wide rows: every thread owns a range of columns and walks all rows (no partial buffers)
    parallel_ranges(D, 64, [=](int64_t c0, int64_t c1) {
      std::vector<double> ag(c1 - c0, 0.0), ab(c1 - c0, 0.0);
      for (int64_t r = 0; r < N; ++r) {
        const T* xr = x + r * D;
        const T* dr = dy + r * D;
        const float m = mean[r], s = rstd[r];
        for (int64_t j = c0; j < c1; ++j) {
          const float d = load_as_float(dr, j);
          ag[j - c0] += static_cast<double>(d) * ((load_as_float(xr, j) - m) * s);
          ab[j - c0] += d;
        }
      }
      for (int64_t j = c0; j < c1; ++j) {
        dgamma[j] = static_cast<float>(ag[j - c0]);
        dbeta[j] = static_cast<float>(ab[j - c0]);
      }
    });
    return;
  }
  const int64_t blocks = std::min<int64_t>(kColumnSumBlocks, N);
  const int64_t rows_per_block = (N + blocks - 1) / blocks;
  std::vector<double> part(static_cast<size_t>(blocks) * 2 * D, 0.0);
  double* pp = part.data();
  parallel_ranges(blocks, rows_per_thread_floor(rows_per_block * D), [=](int64_t b0, int64_t b1) {
    for (int64_t b = b0; b < b1; ++b) {
      double* ag = pp + b * 2 * D;
      double* ab = ag + D;
      const int64_t r_end = std::min<int64_t>(N, (b + 1) * rows_per_block);
      for (int64_t r = b * rows_per_block; r < r_end; ++r) {
        const T* xr = x + r * D;
        const T* dr = dy + r * D;
        const float m = mean[r], s = rstd[r];
        for (int64_t j = 0; j < D; ++j) {
          const float d = load_as_float(dr, j);
          ag[j] += static_cast<double>(d) * ((load_as_float(xr, j) - m) * s);
          ab[j] += d;
        }
      }
    }
  });
  for (int64_t j = 0; j < D; ++j) {
    double g = 0.0, b = 0.0;
    for (int64_t k = 0; k < blocks; ++k) {
      g += pp[k * 2 * D + j];
      b += pp[k * 2 * D + D + j];
    }
    dgamma[j] = static_cast<float>(g);
    dbeta[j] = static_cast<float>(b);
  }
}

// ------------------------------------------------------ InstanceNorm, channel-first [N, C, D]
template <typename T>
void instance_norm_cf_fwd_t(const T* x, const float* gamma, const float* beta, int64_t N, int64_t C,
                            int64_t D, float eps, T* y, float* mean, float* rstd) {
  parallel_ranges(N * C, rows_per_thread_floor(D), [=](int64_t p0, int64_t p1) {
    for (int64_t p = p0; p < p1; ++p) {
      const T* xr = x + p * D;
      T* yr = y + p * D;
      float m, s;
      row_stats(xr, D, eps, &m, &s);
      const float a = s * gamma[p % C], b = beta[p % C];
      for (int64_t j = 0; j < D; ++j) store_from_float(yr, j, (load_as_float(xr, j) - m) * a + b);
      mean[p] = m;
      rstd[p] = s;
    }
  });
}

template <typename T>
void instance_norm_cf_bwd_t(const T* dy, const T* x, const float* gamma, const float* mean,
                            const float* rstd, int64_t N, int64_t C, int64_t D, T* dx,
                            float* dgamma, float* dbeta) {
  // per plane: sum dy and sum dy * xh (they give both the row sums of dx and the plane's share
  // of dgamma / dbeta), kept for the fold over n
  std::vector<double> plane(static_cast<size_t>(N) * C * 2);
  double* pl = plane.data();
  parallel_ranges(N * C, rows_per_thread_floor(D), [=](int64_t p0, int64_t p1) {
    for (int64_t p = p0; p < p1; ++p) {
      double a, b;  // sum dy, sum dy * xh
      row_bwd_sums(dy + p * D, x + p * D, nullptr, 1.0f, mean[p], rstd[p], D, &a, &b);
      pl[2 * p] = a;
      pl[2 * p + 1] = b;
      const float gc = gamma[p % C];
      row_bwd_dx(dy + p * D, x + p * D, nullptr, gc, mean[p], rstd[p], D, a * gc, b * gc, dx + p * D);
    }
  });
  for (int64_t c = 0; c < C; ++c) {
    double g = 0.0, b = 0.0;
    for (int64_t n = 0; n < N; ++n) {
      b += pl[2 * (n * C + c)];
      g += pl[2 * (n * C + c) + 1];
    }
    dgamma[c] = static_cast<float>(g);
    dbeta[c] = static_cast<float>(b);
  }
}

// ------------------------------------------------------- InstanceNorm, channels-last [N, D, C]
// An instance is cut into pixel blocks; every block keeps per-channel accumulators and walks
// its pixels in memory order, the blocks of an instance are then combined in order.  The
// variance comes from a second sweep around the instance mean, as in the channel-first case.
constexpr int64_t kPixelBlocks = 16;

struct ClSplit {
  int64_t blocks, pixels_per_block;
};
inline ClSplit cl_split(int64_t D) {
  ClSplit s;
  s.blocks = std::min<int64_t>(kPixelBlocks, D);
  s.pixels_per_block = (D + s.blocks - 1) / s.blocks;
  return s;
}

// acc[(n * blocks + b) * width + k] += per-channel terms over the pixels of block b of instance n
template <typename Body>
void cl_accumulate(int64_t N, int64_t C, int64_t D, int width, std::vector<double>* acc, Body body) {
  const ClSplit sp = cl_split(D);
  acc->assign(static_cast<size_t>(N) * sp.blocks * width * C, 0.0);
  double* a = acc->data();
  parallel_ranges(N * sp.blocks, std::max<int64_t>(1, kMinElemsPerThread / std::max<int64_t>(1, sp.pixels_per_block * C)),
                  [=](int64_t w0, int64_t w1) {
                    for (int64_t w = w0; w < w1; ++w) {
                      const int64_t n = w / sp.blocks, b = w % sp.blocks;
                      const int64_t p_end = std::min<int64_t>(D, (b + 1) * sp.pixels_per_block);
                      double* out = a + w * width * C;
                      for (int64_t p = b * sp.pixels_per_block; p < p_end; ++p) body(n, p, out);
                    }
                  });
}

// sums[(n * C + c) * width + k] = sum over the blocks of instance n, in block order
void cl_fold_blocks(const std::vector<double>& acc, int64_t N, int64_t C, int64_t D, int width,
                    std::vector<double>* sums) {
  const ClSplit sp = cl_split(D);
  sums->assign(static_cast<size_t>(N) * C * width, 0.0);
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t b = 0; b < sp.blocks; ++b) {
      const double* in = acc.data() + (n * sp.blocks + b) * width * C;
      for (int k = 0; k < width; ++k) {
        for (int64_t c = 0; c < C; ++c) (*sums)[(n * C + c) * width + k] += in[k * C + c];
      }
    }
  }
}

template <typename T>
void instance_norm_cl_fwd_t(const T* x, const float* gamma, const float* beta, int64_t N, int64_t C,
                            int64_t D, float eps, T* y, float* mean, float* rstd) {
  std::vector<double> acc, sums;
  cl_accumulate(N, C, D, 1, &acc, [=](int64_t n, int64_t p, double* out) {
    const T* px = x + (n * D + p) * C;
    for (int64_t c = 0; c < C; ++c) out[c] += load_as_float(px, c);
  });
  cl_fold_blocks(acc, N, C, D, 1, &sums);
  for (int64_t i = 0; i < N * C; ++i) mean[i] = static_cast<float>(sums[i] / static_cast<double>(D));
  cl_accumulate(N, C, D, 1, &acc, [=](int64_t n, int64_t p, double* out) {
    const T* px = x + (n * D + p) * C;
    const float* mn = mean + n * C;
    for (int64_t c = 0; c < C; ++c) {
      const float d = load_as_float(px, c) - mn[c];
      out[c] += static_cast<double>(d) * d;
    }
  });
  cl_fold_blocks(acc, N, C, D, 1, &sums);
  for (int64_t i = 0; i < N * C; ++i) {
    rstd[i] = static_cast<float>(1.0 / std::sqrt(sums[i] / static_cast<double>(D) + static_cast<double>(eps)));
  }
  parallel_ranges(N * D, std::max<int64_t>(1, kMinElemsPerThread / std::max<int64_t>(1, C)),
                  [=](int64_t q0, int64_t q1) {
                    for (int64_t q = q0; q < q1; ++q) {
                      const int64_t n = q / D;
                      const T* px = x + q * C;
                      T* py = y + q * C;
                      const float* mn = mean + n * C;
                      const float* rs = rstd + n * C;
                      for (int64_t c = 0; c < C; ++c) {
                        store_from_float(py, c, (load_as_float(px, c) - mn[c]) * (rs[c] * gamma[c]) + beta[c]);
                      }
                    }
                  });
}

template <typename T>
void instance_norm_cl_bwd_t(const T* dy, const T* x, const float* gamma, const float* mean,
                            const float* rstd, int64_t N, int64_t C, int64_t D, T* dx,
                            float* dgamma, float* dbeta) {
  std::vector<double> acc, sums;  // per (n, c): [0] sum dy, [1] sum dy * xh
  cl_accumulate(N, C, D, 2, &acc, [=](int64_t n, int64_t p, double* out) {
    const T* px = x + (n * D + p) * C;
    const T* pd = dy + (n * D + p) * C;
    const float* mn = mean + n * C;
    const float* rs = rstd + n * C;
    for (int64_t c = 0; c < C; ++c) {
      const float d = load_as_float(pd, c);
      out[c] += d;
      out[C + c] += static_cast<double>(d) * ((load_as_float(px, c) - mn[c]) * rs[c]);
    }
  });
  cl_fold_blocks(acc, N, C, D, 2, &sums);
  for (int64_t c = 0; c < C; ++c) {
    double g = 0.0, b = 0.0;
    for (int64_t n = 0; n < N; ++n) {
      b += sums[(n * C + c) * 2];
      g += sums[(n * C + c) * 2 + 1];
    }
    dgamma[c] = static_cast<float>(g);
    dbeta[c] = static_cast<float>(b);
  }
  const double* sm = sums.data();
  const float inv_d = 1.0f / static_cast<float>(D);
  parallel_ranges(N * D, std::max<int64_t>(1, kMinElemsPerThread / std::max<int64_t>(1, C)),
                  [=](int64_t q0, int64_t q1) {
                    for (int64_t q = q0; q < q1; ++q) {
                      const int64_t n = q / D;
                      const T* px = x + q * C;
                      const T* pd = dy + q * C;
                      T* po = dx + q * C;
                      for (int64_t c = 0; c < C; ++c) {
                        const float m = mean[n * C + c], s = rstd[n * C + c], gc = gamma[c];
                        const float a = static_cast<float>(sm[(n * C + c) * 2]) * gc * inv_d;
                        const float b = static_cast<float>(sm[(n * C + c) * 2 + 1]) * gc * inv_d;
                        const float xh = (load_as_float(px, c) - m) * s;
                        store_from_float(po, c, s * (load_as_float(pd, c) * gc - (a + xh * b)));
                      }
                    }
                  });
}

}  // namespace

// ------------------------------------------------------------------ dtype dispatch
#define ATEXN_CPU_DISPATCH(dtype, CALL)                        \
  switch (dtype) {                                             \
    case 0: { using T = float; CALL; return true; }            \
    case 1: { using T = Half; CALL; return true; }             \
    case 2: { using T = BFloat16; CALL; return true; }         \
    default: return false;                                     \
  }

bool layer_norm_fwd(int dtype, const void* x, const float* gamma, const float* beta, int64_t N,
                    int64_t D, float eps, void* y, float* mean, float* rstd) {
  ATEXN_CPU_DISPATCH(dtype, layer_norm_fwd_t<T>(static_cast<const T*>(x), gamma, beta, N, D, eps,
                                                static_cast<T*>(y), mean, rstd));
}

bool layer_norm_bwd(int dtype, const void* dy, const void* x, const float* gamma, const float* mean,
                    const float* rstd, int64_t N, int64_t D, void* dx, float* dgamma, float* dbeta) {
  ATEXN_CPU_DISPATCH(dtype, layer_norm_bwd_t<T>(static_cast<const T*>(dy), static_cast<const T*>(x), gamma,
                                                mean, rstd, N, D, static_cast<T*>(dx), dgamma, dbeta));
}

bool instance_norm_fwd(int dtype, bool channel_first, const void* x, const float* gamma,
                       const float* beta, int64_t N, int64_t C, int64_t D, float eps, void* y,
                       float* mean, float* rstd) {
  if (channel_first) {
    ATEXN_CPU_DISPATCH(dtype, instance_norm_cf_fwd_t<T>(static_cast<const T*>(x), gamma, beta, N, C, D, eps,
                                                        static_cast<T*>(y), mean, rstd));
  }
  ATEXN_CPU_DISPATCH(dtype, instance_norm_cl_fwd_t<T>(static_cast<const T*>(x), gamma, beta, N, C, D, eps,
                                                      static_cast<T*>(y), mean, rstd));
}

bool instance_norm_bwd(int dtype, bool channel_first, const void* dy, const void* x,
                       const float* gamma, const float* mean, const float* rstd, int64_t N,
                       int64_t C, int64_t D, void* dx, float* dgamma, float* dbeta) {
  if (channel_first) {
    ATEXN_CPU_DISPATCH(dtype, instance_norm_cf_bwd_t<T>(static_cast<const T*>(dy), static_cast<const T*>(x),
                                                        gamma, mean, rstd, N, C, D, static_cast<T*>(dx),
                                                        dgamma, dbeta));
  }
  ATEXN_CPU_DISPATCH(dtype, instance_norm_cl_bwd_t<T>(static_cast<const T*>(dy), static_cast<const T*>(x),
                                                      gamma, mean, rstd, N, C, D, static_cast<T*>(dx),
                                                      dgamma, dbeta));
}

}  // namespace cpu
}  // namespace atexn
