// extern "C" surface of libatex_norms_hip.so (declared in include/atex_norms.h).
//
// Kernel level: argument validation + routing to the row / channels-last launchers.
// Op level: the host logic of the reference's OpKernel::Compute methods
// (cc/kernels/fused_layer_norm_op.cc:295-352, :370-458;
//  cc/kernels/fused_instance_norm_op.cc:328-406, :430-534) minus tensor allocation,
// which stays with the caller.
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <exception>
#include <mutex>
#include <vector>

#include "cpu_kernels.h"
#include "plan.h"
#include "status.h"
#ifdef ATEXN_BENCH_BUILD
#include "bench_hooks.h"
#endif

using namespace atexn;

// Device scratch of atexn_layer_norm_bwd_static: part of the library's code object, so every
// GPU the library runs on holds its own copy from module load until the process ends.  In host
// code the array's name is only a handle; its device address comes from hipGetSymbolAddress,
// once per device, and only that address is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[ATEXN_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kAbiVersion = 2;
constexpr int64_t kMaxInt = 2147483647;

bool dtype_ok(int dtype) { return dtype == ATEXN_F32 || dtype == ATEXN_F16 || dtype == ATEXN_BF16; }
bool ws_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 255u) == 0; }

int64_t num_elements(const atexn_tensor* t) {
  int64_t n = 1;
  for (int i = 0; i < t->rank; ++i) n *= t->dims[i];
  return n;
}

bool same_shape(const atexn_tensor* a, const atexn_tensor* b) {
  if (a->rank != b->rank) return false;
  for (int i = 0; i < a->rank; ++i)
    if (a->dims[i] != b->dims[i]) return false;
  return true;
}

int check_tensor(const atexn_tensor* t, const char* name) {
  ATEXN_REQUIRE(t != nullptr, "%s is NULL", name);
  ATEXN_REQUIRE(t->rank >= 0 && t->rank <= ATEXN_MAX_RANK, "%s has unsupported rank %d", name, t->rank);
  for (int i = 0; i < t->rank; ++i)
    ATEXN_REQUIRE(t->dims[i] >= 0, "%s has negative dim %lld", name, (long long)t->dims[i]);
  ATEXN_REQUIRE(num_elements(t) == 0 || t->data != nullptr, "%s has elements but a NULL data pointer", name);
  return ATEXN_OK;
}

bool device_ok(const atexn_tensor* t) {
  return t->device == ATEXN_DEVICE_GPU || t->device == ATEXN_DEVICE_CPU;
}

// All tensors of a call on the device of the first one.
template <typename... Ts>
int check_same_device(const atexn_tensor* first, const Ts*... rest) {
  ATEXN_REQUIRE(device_ok(first), "bad device %d", first->device);
  const atexn_tensor* all[] = {rest...};
  for (const atexn_tensor* t : all) {
    ATEXN_REQUIRE(t->device == first->device,
                  "all tensors of an op must be on the same device (got %d and %d)", first->device,
                  t->device);
  }
  return ATEXN_OK;
}

#define ATEXN_TRY(expr)             \
  do {                              \
    int s_ = (expr);                \
    if (s_ != ATEXN_OK) return s_;  \
  } while (0)

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the current device: looked up once per device (under the lock), read
// with one atomic load afterwards.
int static_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error(ATEXN_LAUNCH_ERROR, "hipGetDevice: %s", hipGetErrorString(e));
  ATEXN_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d not supported (limit %d)", dev,
                kMaxDevices);
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (p == nullptr) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || p == nullptr) {
        (void)hipGetLastError();
        return set_error(ATEXN_LAUNCH_ERROR, "hipGetSymbolAddress(scratch) on device %d: %s", dev,
                         hipGetErrorString(e));
      }
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *out = p;
  return ATEXN_OK;
}

// The host kernels start threads and allocate: whatever they throw (std::system_error when a
// thread cannot be created, std::bad_alloc) stops here and becomes a status.
template <typename F>
int guarded_cpu_call(const char* what, F&& f) {
  try {
    f();
  } catch (const std::exception& e) {
    return set_error(ATEXN_LAUNCH_ERROR, "%s: %s", what, e.what());
  } catch (...) {
    return set_error(ATEXN_LAUNCH_ERROR, "%s: unknown exception", what);
  }
  return ATEXN_OK;
}

}  // namespace

extern "C" {

const char* atexn_status_string(int status) {
  switch (status) {
    case ATEXN_OK: return "OK";
    case ATEXN_INVALID_ARGUMENT: return "INVALID_ARGUMENT";
    case ATEXN_LAUNCH_ERROR: return "LAUNCH_ERROR";
    default: return "UNKNOWN";
  }
}

const char* atexn_last_error(void) { return last_error(); }
int atexn_abi_version(void) { return kAbiVersion; }

#ifdef ATEXN_BENCH_BUILD
/* ------------------------------------------------------ benchmark build only (bench_hooks.h) */

/* Sets a launch-planning parameter by name for the whole process.  Returns
 * ATEXN_INVALID_ARGUMENT for an unknown name or a value out of range.  Every setting but
 * bwd_stage_mask != 3 computes complete, correct results. */
int atexn_set_tuning(const char* name, int value) {
  ATEXN_REQUIRE(name != nullptr && value >= 0, "bad tuning request");
  ATEXN_REQUIRE(value >= 1 || !strcmp(name, "reverse_second_pass") || !strcmp(name, "cl_fused") ||
                    !strcmp(name, "cl_fold_cap") || !strcmp(name, "cl_single") || !strcmp(name, "affine_fold") || !strcmp(name, "affine_fold_polls") || !strcmp(name, "cl_single_polls") || !strcmp(name, "cl_single_xm") || !strcmp(name, "cl_single_occ") || !strcmp(name, "plane_single") || !strcmp(name, "plane_single_occ") || !strcmp(name, "plane_single_polls") || !strcmp(name, "bwd_lds_rows") || !strcmp(name, "staged_rows") || !strcmp(name, "cl_narrow_tiles") || !strcmp(name, "cl_fused_split"),
                "value must be >= 1");
  Tuning& t = tuning();
  if (!strcmp(name, "fwd_waves_per_cu")) t.fwd_waves_per_cu = value;
  else if (!strcmp(name, "bwd_ln_threads")) {
    ATEXN_REQUIRE(value == 256 || value == 512, "bwd_ln_threads must be 256 or 512");
    t.bwd_ln_threads = value;
  } else if (!strcmp(name, "bwd_waves_per_cu")) t.bwd_waves_per_cu = value;
  else if (!strcmp(name, "bwd_affine_waves_per_cu")) t.bwd_affine_waves_per_cu = value;
  else if (!strcmp(name, "bwd_min_rows")) t.bwd_min_rows = value;
  else if (!strcmp(name, "bwd_lds_vpt")) {
    ATEXN_REQUIRE(value == 4 || value == 8, "bwd_lds_vpt must be 4 or 8");
    t.bwd_lds_vpt = value;
  }
  else if (!strcmp(name, "staged_rows")) {
    ATEXN_REQUIRE(value >= 0 && value <= 2, "staged_rows must be 0, 1 or 2");
    t.staged_rows = value;
  } else if (!strcmp(name, "bwd_lds_rows")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "bwd_lds_rows must be 0 or 1");
    t.bwd_lds_rows = value;
  }
  else if (!strcmp(name, "split_items_per_cu")) t.split_items_per_cu = value;
  else if (!strcmp(name, "split_bwd_items_per_cu")) t.split_bwd_items_per_cu = value;
  else if (!strcmp(name, "cl_items_per_cu")) t.cl_items_per_cu = value;
  else if (!strcmp(name, "cl_bwd_big_items")) t.cl_bwd_big_items = value;
  else if (!strcmp(name, "tile_items_per_cu")) t.tile_items_per_cu = value;
  else if (!strcmp(name, "fwd_rows_batch_v1")) {
    ATEXN_REQUIRE(value == 1 || value == 2 || value == 4, "fwd_rows_batch_v1 must be 1, 2 or 4");
    t.fwd_rows_batch_v1 = value;
  } else if (!strcmp(name, "fwd_rows_batch") || !strcmp(name, "bwd_rows_batch")) {
    ATEXN_REQUIRE(value == 1 || value == 2 || (value == 4 && name[0] == 'f'),
                  "rows batch must be 1, 2 (or 4, forward only)");
    (name[0] == 'f' ? t.fwd_rows_batch : t.bwd_rows_batch) = value;
  } else if (!strcmp(name, "bwd_stage_mask")) {
    ATEXN_REQUIRE(value >= 1 && value <= 3, "bwd_stage_mask must be 1, 2 or 3");
    t.bwd_stage_mask = value;
  } else if (!strcmp(name, "bwd_wave_groups")) {
    ATEXN_REQUIRE(value == 1 || value == 2, "bwd_wave_groups must be 1 (on) or 2 (off)");
    t.bwd_wave_groups = value == 1;
  } else if (!strcmp(name, "fwd_vpt2_max_vec")) {
    ATEXN_REQUIRE(value >= 1024 && value <= 2048, "fwd_vpt2_max_vec must be in [1024, 2048]");
    t.fwd_vpt2_max_vec = value;
  } else if (!strcmp(name, "fwd_vpt4_max_vec")) {
    ATEXN_REQUIRE(value >= 2048 && value <= 3072, "fwd_vpt4_max_vec must be in [2048, 3072]");
    t.fwd_vpt4_max_vec = value;
  } else if (!strcmp(name, "bwd_vpt2_max_vec")) {
    ATEXN_REQUIRE(value >= 1024 && value <= 1536, "bwd_vpt2_max_vec must be in [1024, 1536]");
    t.bwd_vpt2_max_vec = value;
  } else if (!strcmp(name, "cl_fused")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_fused must be 0 or 1");
    t.cl_fused = value;
  } else if (!strcmp(name, "cl_fused_split")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_fused_split must be 0 or 1");
    t.cl_fused_split = value;
  } else if (!strcmp(name, "cl_narrow_tiles")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_narrow_tiles must be 0 or 1");
    t.cl_narrow_tiles = value;
  } else if (!strcmp(name, "affine_fold")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "affine_fold must be 0 or 1");
    t.affine_fold = value;
  } else if (!strcmp(name, "affine_fold_polls")) {
    t.affine_fold_polls = value;
  } else if (!strcmp(name, "plane_single")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "plane_single must be 0 or 1");
    t.plane_single = value;
  } else if (!strcmp(name, "plane_single_polls")) {
    t.plane_single_polls = value;
  } else if (!strcmp(name, "plane_single_occ")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "plane_single_occ must be 0 or 1");
    t.plane_single_occ = value;
  } else if (!strcmp(name, "plane_nt_min_mb")) {
    t.plane_nt_min_mb = value;
  } else if (!strcmp(name, "cl_single")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_single must be 0 or 1");
    t.cl_single = value;
  } else if (!strcmp(name, "cl_single_xm")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_single_xm must be 0 or 1");
    t.cl_single_xm = value;
  } else if (!strcmp(name, "cl_single_occ")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_single_occ must be 0 or 1");
    t.cl_single_occ = value;
  } else if (!strcmp(name, "cl_single_polls")) {
    t.cl_single_polls = value;
  } else if (!strcmp(name, "cl_fold_cap")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "cl_fold_cap must be 0 or 1");
    t.cl_fold_cap = value;
  } else if (!strcmp(name, "reverse_second_pass")) {
    ATEXN_REQUIRE(value == 0 || value == 1, "reverse_second_pass must be 0 or 1");
    t.reverse_second_pass = value;
  }
  else return set_error(ATEXN_INVALID_ARGUMENT, "unknown tuning parameter '%s'", name);
  return ATEXN_OK;
}

/* Which kernels a backward call of this shape launches, as text: the row / plane kernel family,
 * its launch geometry, and whether a separate column reduction follows (the part that
 * bwd_stage_mask = 1 leaves out).  op: 0 LayerNorm [N, D] (C ignored), 1 InstanceNorm.  Returns
 * the length written (0 on a bad argument). */
int atexn_bench_describe_bwd(int op, int dtype, int layout, int64_t N, int64_t C, int64_t D,
                             char* out, size_t out_bytes) {
  if (!out || out_bytes == 0 || !dtype_ok(dtype) || N <= 0 || D <= 0 || (op == 1 && C <= 0)) return 0;
  const int vec = 16 / elem_size(dtype);
  const int cus = cu_count();
  int n = 0;
  if (op == 1 && layout == ATEXN_LAYOUT_N_C) {
    const ClPlan p = plan_cl(true, C >= vec ? vec : 1, N, C, D, cus);
    if (p.fused)
      n = snprintf(out, out_bytes, "cl_bwd_fused (u=%d, grid %lld x %d)%s; alone=0", p.fused_u, (long long)N,
                   p.CT, N > 1 ? " + col_reduce" : "");
    else if (p.single)
      n = snprintf(out, out_bytes, "cl_bwd_single (S=%d slabs, tiles=%d, U=%d%s; two stages when dx == dy or under capture)%s; alone=0",
                   p.S, p.CT, p.U, p.single_xm ? ", XCD-major grid" : "", p.single_xm && !p.xm_fold && N > 1 ? " + col_reduce" : "");
    else
      n = snprintf(out, out_bytes, "cl_bwd_sums + %scl_bwd_apply (S=%d slabs, tiles=%d, U=%d); alone=0",
                   p.fold ? "col_reduce + " : "", p.S, p.CT, p.U);
  } else {
    const bool affine = op == 1;
    const RowsKind kind = affine ? RowsKind::kBwdAffine : RowsKind::kBwdCols;
    const int64_t rows = affine ? N * C : N;
    const RowsRoute r = route_rows(kind, !affine, vec, rows, D);
    if (r.small) {
      n = snprintf(out, out_bytes, "small_bwd + col_reduce; alone=1");
    } else if (r.tiles) {
      const TilePlan p = plan_tiles(true, vec, rows, D, cus);
      n = snprintf(out, out_bytes, "tile_bwd_sums + merge_row_sums + tile_bwd_apply%s; alone=0",
                   p.sums_RS > 1 ? " + col_reduce" : "");
    } else {
      const RowsPlan p = plan_rows(kind, r.V, rows, D, affine ? static_cast<int>(C) : 0, cus);
      const char* k = p.acc_lds ? "rows_bwd_lds" : p.staged ? "rows_bwd_staged" : p.resident ? "rows_bwd_resident" : "";
      const char* two = p.staged ? "rows_bwd_staged" : "split_bwd_sums + split_bwd_apply";
      if (p.plane_single)
        n = snprintf(out, out_bytes, "plane_bwd_single (S=%d chunks of %d vectors, grid %d x %d threads; %s when dx == dy or under capture)%s; alone=0",
                     p.ps_S, p.ps_chunk_vec, p.ps_grid, kPlanPlaneThreads, two,
                     p.ps_fold ? ", plane sums folded over the batch in the kernel" : " + col_reduce");
      else if (k[0] && p.affine_fold)
        n = snprintf(out, out_bytes, "%s (grid %d x %d threads, tpr=%d vpt=%d rb=%d), plane sums folded over the batch in the kernel (col_reduce follows instead when dx == dy or under capture); alone=0",
                     k, p.grid, p.threads, p.tpr, p.vpt, p.rb);
      else if (k[0])
        n = snprintf(out, out_bytes, "%s (grid %d x %d threads, tpr=%d vpt=%d rb=%d) + col_reduce over %d partial rows; alone=1",
                     k, p.grid, p.threads, p.tpr, p.vpt, p.rb, p.part_rows);
      else
        n = snprintf(out, out_bytes, "split_bwd_sums + split_bwd_apply (S=%d chunks) + col_reduce; alone=0", p.S);
    }
  }
  return n < 0 ? 0 : (static_cast<size_t>(n) < out_bytes ? n : static_cast<int>(out_bytes) - 1);
}

int atexn_bench_mark_exchange_trouble(int recent) {
  unsigned* word = exchange_trouble_word();
  ATEXN_REQUIRE(word != nullptr, "no record of waits on this device");
  const unsigned value = next_call_tag() - (recent ? 0u : 0x40000000u);
  const hipError_t e = hipMemcpy(word, &value, sizeof(value), hipMemcpyHostToDevice);
  if (e != hipSuccess) return set_error(ATEXN_LAUNCH_ERROR, "hipMemcpy: %s", hipGetErrorString(e));
  return ATEXN_OK;
}

namespace {
// Holds a whole CU per workgroup (its LDS) until the wall clock (100 MHz) has advanced by `ticks`
// or `max_passes` loop passes are over, whichever comes first: it cannot outstay its bound.
__global__ void __launch_bounds__(1024) occupy_kernel(long long ticks, int max_passes, int* sink) {
  extern __shared__ int occupy_pad[];
  const long long t0 = wall_clock64();
  int v = threadIdx.x;
  for (int pass = 0; pass < max_passes && wall_clock64() - t0 < ticks; ++pass) {
    v = v * 1664525 + 1013904223;
    __builtin_amdgcn_s_sleep(20);
  }
  occupy_pad[threadIdx.x] = v;
  if (sink != nullptr && v == 0x7fffffff) sink[0] = occupy_pad[0];
}
}  // namespace

int atexn_bench_occupy(int workgroups, double milliseconds, void* stream) {
  ATEXN_REQUIRE(workgroups >= 1 && workgroups <= 1024, "1 to 1024 workgroups");
  ATEXN_REQUIRE(milliseconds > 0.0 && milliseconds <= 100.0, "at most 100 milliseconds");
  constexpr int kLds = 158 * 1024;  // of a CU's 160 KB: no workgroup of another kernel fits beside it
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(occupy_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
  if (e != hipSuccess) return set_error(ATEXN_LAUNCH_ERROR, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  // a pass is a sleep of about 0.6 us: the cap is some ten times the time asked for
  const int max_passes = static_cast<int>(milliseconds * 20000.0) + 1000;
  occupy_kernel<<<workgroups, 1024, kLds, static_cast<hipStream_t>(stream)>>>(
      static_cast<long long>(milliseconds * 1e5), max_passes, nullptr);
  e = hipGetLastError();
  if (e != hipSuccess) return set_error(ATEXN_LAUNCH_ERROR, "occupy_kernel: %s", hipGetErrorString(e));
  return ATEXN_OK;
}

int atexn_bench_exchange_trouble_age(void) {
  unsigned* word = exchange_trouble_word();
  unsigned value = 0;
  if (word == nullptr || hipDeviceSynchronize() != hipSuccess ||
      hipMemcpy(&value, word, sizeof(value), hipMemcpyDeviceToHost) != hipSuccess) {
    (void)hipGetLastError();
    return -1;
  }
  const unsigned age = next_call_tag() - value;
  return age > 0x7fffffffu ? 0x7fffffff : static_cast<int>(age);
}
#endif  // ATEXN_BENCH_BUILD

/* ------------------------------------------------------------------ kernel level */

size_t atexn_layer_norm_fwd_workspace_bytes(int dtype, int64_t N, int64_t D) {
  if (!dtype_ok(dtype)) return 0;
  return rows_fwd_ws(dtype, false, N, D, 1);
}

int atexn_layer_norm_fwd(int dtype, const void* x, const float* gamma, const float* beta,
                         int64_t N, int64_t D, float epsilon, void* y, float* mean,
                         float* inv_std, void* workspace, size_t workspace_bytes,
                         void* stream) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(N >= 0 && D >= 0, "negative size N=%lld D=%lld", (long long)N, (long long)D);
  if (N == 0 || D == 0) return ATEXN_OK;
  ATEXN_REQUIRE(x && gamma && beta && y && mean && inv_std, "NULL pointer argument");
  ATEXN_REQUIRE(workspace == nullptr || ws_aligned(workspace), "workspace must be 256-byte aligned");
  return rows_fwd(dtype, false, x, gamma, beta, N, D, 1, epsilon, y, mean, inv_std, workspace,
                  workspace_bytes, static_cast<hipStream_t>(stream));
}

size_t atexn_layer_norm_bwd_workspace_bytes(int dtype, int64_t N, int64_t D) {
  if (!dtype_ok(dtype)) return 0;
  return rows_bwd_ws(dtype, false, N, D, 1);
}

int atexn_layer_norm_bwd(int dtype, const void* dy, const void* x, const float* gamma,
                         const float* mean, const float* inv_std, int64_t N, int64_t D,
                         void* dx, float* dgamma, float* dbeta, void* workspace,
                         size_t workspace_bytes, void* stream) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(N >= 0 && D >= 0, "negative size N=%lld D=%lld", (long long)N, (long long)D);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (N == 0 || D == 0) {
    if (D > 0) {
      ATEXN_REQUIRE(dgamma && dbeta, "NULL pointer argument");
      ATEXN_TRY(fill_zero(dgamma, D, st));
      ATEXN_TRY(fill_zero(dbeta, D, st));
    }
    return ATEXN_OK;
  }
  ATEXN_REQUIRE(dy && x && gamma && mean && inv_std && dx && dgamma && dbeta, "NULL pointer argument");
  ATEXN_REQUIRE(dx != x, "dx must not alias x (it may alias dy)");
  ATEXN_REQUIRE(workspace != nullptr && ws_aligned(workspace), "workspace must be non-NULL and 256-byte aligned");
  return rows_bwd(dtype, false, dy, x, gamma, mean, inv_std, N, D, 1, dx, dgamma, dbeta, workspace,
                  workspace_bytes, st);
}

int atexn_layer_norm_bwd_static(int dtype, const void* dy, const void* x, const float* gamma,
                                const float* mean, const float* inv_std, int64_t N, int64_t D,
                                void* dx, float* dgamma, float* dbeta, void* stream) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(N >= 0 && D >= 0, "negative size N=%lld D=%lld", (long long)N, (long long)D);
  const size_t need = rows_bwd_ws(dtype, false, N, D, 1);
  ATEXN_REQUIRE(need <= sizeof(scratch),
                "LayerNorm backward of [%lld, %lld] needs %zu bytes of scratch, more than the %zu "
                "bytes of the static buffer: use atexn_layer_norm_bwd with a workspace",
                (long long)N, (long long)D, need, sizeof(scratch));
  void* ws = nullptr;
  if (need > 0) ATEXN_TRY(static_scratch(&ws));
  // the kernels overwrite every scratch word they later read (one partial dgamma / dbeta row
  // per workgroup, per-row sums), so nothing has to be cleared between calls
  return atexn_layer_norm_bwd(dtype, dy, x, gamma, mean, inv_std, N, D, dx, dgamma, dbeta, ws,
                              sizeof(scratch), stream);
}

size_t atexn_instance_norm_fwd_workspace_bytes(int dtype, int layout, int64_t N, int64_t C,
                                               int64_t D) {
  if (!dtype_ok(dtype) || N <= 0 || C <= 0 || D <= 0 || C > kMaxInt || N > kMaxInt) return 0;
  return layout == ATEXN_LAYOUT_NC_ ? rows_fwd_ws(dtype, true, N * C, D, static_cast<int>(C))
                                    : cl_fwd_ws(dtype, N, C, D);
}

int atexn_instance_norm_fwd(int dtype, int layout, const void* x, const float* gamma,
                            const float* beta, int64_t N, int64_t C, int64_t D,
                            float epsilon, void* y, float* mean, float* inv_std,
                            void* workspace, size_t workspace_bytes, void* stream) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(layout == ATEXN_LAYOUT_NC_ || layout == ATEXN_LAYOUT_N_C, "bad layout %d", layout);
  ATEXN_REQUIRE(N >= 0 && C >= 0 && D >= 0, "negative size");
  ATEXN_REQUIRE(C <= kMaxInt && N <= kMaxInt, "N=%lld or C=%lld too large", (long long)N, (long long)C);
  if (N == 0 || C == 0 || D == 0) return ATEXN_OK;
  ATEXN_REQUIRE(x && gamma && beta && y && mean && inv_std, "NULL pointer argument");
  ATEXN_REQUIRE(workspace == nullptr || ws_aligned(workspace), "workspace must be 256-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (layout == ATEXN_LAYOUT_NC_) {
    return rows_fwd(dtype, true, x, gamma, beta, N * C, D, static_cast<int>(C), epsilon, y, mean,
                    inv_std, workspace, workspace_bytes, st);
  }
  return cl_fwd(dtype, x, gamma, beta, N, C, D, epsilon, y, mean, inv_std, workspace,
                workspace_bytes, st);
}

size_t atexn_instance_norm_bwd_workspace_bytes(int dtype, int layout, int64_t N, int64_t C,
                                               int64_t D) {
  if (!dtype_ok(dtype) || N <= 0 || C <= 0 || D <= 0 || C > kMaxInt || N > kMaxInt) return 0;
  return layout == ATEXN_LAYOUT_NC_ ? rows_bwd_ws(dtype, true, N * C, D, static_cast<int>(C))
                                    : cl_bwd_ws(dtype, N, C, D);
}

int atexn_instance_norm_bwd(int dtype, int layout, const void* dy, const void* x,
                            const float* gamma, const float* mean, const float* inv_std,
                            int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
                            float* dbeta, void* workspace, size_t workspace_bytes,
                            void* stream) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(layout == ATEXN_LAYOUT_NC_ || layout == ATEXN_LAYOUT_N_C, "bad layout %d", layout);
  ATEXN_REQUIRE(N >= 0 && C >= 0 && D >= 0, "negative size");
  ATEXN_REQUIRE(C <= kMaxInt && N <= kMaxInt, "N=%lld or C=%lld too large", (long long)N, (long long)C);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (N == 0 || C == 0 || D == 0) {
    if (C > 0) {
      ATEXN_REQUIRE(dgamma && dbeta, "NULL pointer argument");
      ATEXN_TRY(fill_zero(dgamma, C, st));
      ATEXN_TRY(fill_zero(dbeta, C, st));
    }
    return ATEXN_OK;
  }
  ATEXN_REQUIRE(dy && x && gamma && mean && inv_std && dx && dgamma && dbeta, "NULL pointer argument");
  ATEXN_REQUIRE(dx != x, "dx must not alias x (it may alias dy)");
  ATEXN_REQUIRE(workspace != nullptr && ws_aligned(workspace), "workspace must be non-NULL and 256-byte aligned");
  if (layout == ATEXN_LAYOUT_NC_) {
    return rows_bwd(dtype, true, dy, x, gamma, mean, inv_std, N * C, D, static_cast<int>(C), dx,
                    dgamma, dbeta, workspace, workspace_bytes, st);
  }
  return cl_bwd(dtype, dy, x, gamma, mean, inv_std, N, C, D, dx, dgamma, dbeta, workspace,
                workspace_bytes, st);
}

/* ------------------------------------------------------------- kernel level, host memory */

int atexn_layer_norm_fwd_cpu(int dtype, const void* x, const float* gamma, const float* beta,
                             int64_t N, int64_t D, float epsilon, void* y, float* mean,
                             float* inv_std) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(N >= 0 && D >= 0, "negative size N=%lld D=%lld", (long long)N, (long long)D);
  if (N == 0 || D == 0) return ATEXN_OK;
  ATEXN_REQUIRE(x && gamma && beta && y && mean && inv_std, "NULL pointer argument");
  return guarded_cpu_call("layer_norm_fwd_cpu", [&] {
    cpu::layer_norm_fwd(dtype, x, gamma, beta, N, D, epsilon, y, mean, inv_std);
  });
}

int atexn_layer_norm_bwd_cpu(int dtype, const void* dy, const void* x, const float* gamma,
                             const float* mean, const float* inv_std, int64_t N, int64_t D,
                             void* dx, float* dgamma, float* dbeta) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(N >= 0 && D >= 0, "negative size N=%lld D=%lld", (long long)N, (long long)D);
  if (N == 0 || D == 0) {
    if (D > 0) {
      ATEXN_REQUIRE(dgamma && dbeta, "NULL pointer argument");
      std::fill(dgamma, dgamma + D, 0.f);
      std::fill(dbeta, dbeta + D, 0.f);
    }
    return ATEXN_OK;
  }
  ATEXN_REQUIRE(dy && x && gamma && mean && inv_std && dx && dgamma && dbeta, "NULL pointer argument");
  ATEXN_REQUIRE(dx != x, "dx must not alias x (it may alias dy)");
  return guarded_cpu_call("layer_norm_bwd_cpu", [&] {
    cpu::layer_norm_bwd(dtype, dy, x, gamma, mean, inv_std, N, D, dx, dgamma, dbeta);
  });
}

int atexn_instance_norm_fwd_cpu(int dtype, int layout, const void* x, const float* gamma,
                                const float* beta, int64_t N, int64_t C, int64_t D,
                                float epsilon, void* y, float* mean, float* inv_std) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(layout == ATEXN_LAYOUT_NC_ || layout == ATEXN_LAYOUT_N_C, "bad layout %d", layout);
  ATEXN_REQUIRE(N >= 0 && C >= 0 && D >= 0, "negative size");
  if (N == 0 || C == 0 || D == 0) return ATEXN_OK;
  ATEXN_REQUIRE(x && gamma && beta && y && mean && inv_std, "NULL pointer argument");
  return guarded_cpu_call("instance_norm_fwd_cpu", [&] {
    cpu::instance_norm_fwd(dtype, layout == ATEXN_LAYOUT_NC_, x, gamma, beta, N, C, D, epsilon, y, mean,
                           inv_std);
  });
}

int atexn_instance_norm_bwd_cpu(int dtype, int layout, const void* dy, const void* x,
                                const float* gamma, const float* mean, const float* inv_std,
                                int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
                                float* dbeta) {
  ATEXN_REQUIRE(dtype_ok(dtype), "bad dtype %d", dtype);
  ATEXN_REQUIRE(layout == ATEXN_LAYOUT_NC_ || layout == ATEXN_LAYOUT_N_C, "bad layout %d", layout);
  ATEXN_REQUIRE(N >= 0 && C >= 0 && D >= 0, "negative size");
  if (N == 0 || C == 0 || D == 0) {
    if (C > 0) {
      ATEXN_REQUIRE(dgamma && dbeta, "NULL pointer argument");
      std::fill(dgamma, dgamma + C, 0.f);
      std::fill(dbeta, dbeta + C, 0.f);
    }
    return ATEXN_OK;
  }
  ATEXN_REQUIRE(dy && x && gamma && mean && inv_std && dx && dgamma && dbeta, "NULL pointer argument");
  ATEXN_REQUIRE(dx != x, "dx must not alias x (it may alias dy)");
  return guarded_cpu_call("instance_norm_bwd_cpu", [&] {
    cpu::instance_norm_bwd(dtype, layout == ATEXN_LAYOUT_NC_, dy, x, gamma, mean, inv_std, N, C, D, dx,
                           dgamma, dbeta);
  });
}

/* ---------------------------------------------------------------------- op level */

int atexn_layer_norm_resolve_axes(int rank, const int64_t* dims, const int* axis, int n_axis,
                                  int64_t* N, int64_t* D) {
  ATEXN_REQUIRE(rank >= 1 && rank <= ATEXN_MAX_RANK, "input must be at least 1-dimensional (rank %d)", rank);
  ATEXN_REQUIRE(dims != nullptr && N != nullptr && D != nullptr, "NULL pointer argument");
  /* an empty axis list is undefined behaviour in the reference (it indexes element 0 of an
   * empty vector, norm_ops.cc:38); rejected here */
  ATEXN_REQUIRE(axis != nullptr && n_axis >= 1, "axis must not be empty");
  std::vector<int> ax;
  for (int i = 0; i < n_axis; ++i) {
    const int a = axis[i] < 0 ? rank + axis[i] : axis[i];
    ATEXN_REQUIRE(a >= 0 && a < rank, "axis contains invalid value: %d", axis[i]);
    ax.push_back(a);
  }
  std::sort(ax.begin(), ax.end());
  ax.erase(std::unique(ax.begin(), ax.end()), ax.end());
  ATEXN_REQUIRE(ax[0] == rank - static_cast<int>(ax.size()), "axis is not packed from last dim.");
  int64_t n = 1, d = 1;
  for (int i = 0; i < rank; ++i) {
    ATEXN_REQUIRE(dims[i] >= 0, "negative dim");
    if (i >= ax[0]) d *= dims[i]; else n *= dims[i];
  }
  *N = n;
  *D = d;
  return ATEXN_OK;
}

int atexn_instance_norm_resolve_format(int rank, const int64_t* dims, const char* data_format,
                                       int* layout, int64_t* N, int64_t* C, int64_t* D) {
  ATEXN_REQUIRE(dims != nullptr && layout && N && C && D, "NULL pointer argument");
  ATEXN_REQUIRE(rank >= 4 && rank <= ATEXN_MAX_RANK, "input must be at least 4-dimensional (rank %d)", rank);
  bool channel_first = false;
  if (data_format != nullptr) {
    const size_t n = strlen(data_format);
    const bool ok = n > 2 && data_format[0] == 'N' && (data_format[1] == 'C' || data_format[n - 1] == 'C');
    ATEXN_REQUIRE(ok, "We only accept 'NC...' or 'N...C' data format, but got %s", data_format);
    channel_first = data_format[1] == 'C';
  }
  int64_t d = 1;
  const int c_dim = channel_first ? 1 : rank - 1;
  const int first = channel_first ? 2 : 1;
  const int last = channel_first ? rank : rank - 1;
  for (int i = first; i < last; ++i) d *= dims[i];
  *layout = channel_first ? ATEXN_LAYOUT_NC_ : ATEXN_LAYOUT_N_C;
  *N = dims[0];
  *C = dims[c_dim];
  *D = d;
  return ATEXN_OK;
}

size_t atexn_fused_layer_norm_workspace_bytes(const atexn_tensor* x, const int* axis, int n_axis) {
  int64_t N, D;
  if (!x || atexn_layer_norm_resolve_axes(x->rank, x->dims, axis, n_axis, &N, &D) != ATEXN_OK) return 0;
  if (x->device == ATEXN_DEVICE_CPU) return 0;
  return atexn_layer_norm_fwd_workspace_bytes(x->dtype, N, D);
}

int atexn_fused_layer_norm(const atexn_tensor* x, const atexn_tensor* scale,
                           const atexn_tensor* offset, float epsilon, const int* axis,
                           int n_axis, atexn_tensor* y, atexn_tensor* reserve_space_1,
                           atexn_tensor* reserve_space_2, void* workspace,
                           size_t workspace_bytes, void* stream) {
  ATEXN_TRY(check_tensor(x, "x"));
  ATEXN_TRY(check_tensor(scale, "scale"));
  ATEXN_TRY(check_tensor(offset, "offset"));
  ATEXN_TRY(check_tensor(y, "y"));
  ATEXN_TRY(check_tensor(reserve_space_1, "reserve_space_1"));
  ATEXN_TRY(check_tensor(reserve_space_2, "reserve_space_2"));
  ATEXN_TRY(check_same_device(x, scale, offset, y, reserve_space_1, reserve_space_2));
  ATEXN_REQUIRE(scale->dtype == ATEXN_F32 && offset->dtype == ATEXN_F32 &&
                    reserve_space_1->dtype == ATEXN_F32 && reserve_space_2->dtype == ATEXN_F32,
                "scale, offset and the reserve spaces must be float32");
  ATEXN_REQUIRE(x->rank > 0, "input must be at least 1-dimensional");
  int64_t N, D;
  ATEXN_TRY(atexn_layer_norm_resolve_axes(x->rank, x->dims, axis, n_axis, &N, &D));
  ATEXN_REQUIRE(num_elements(scale) == D,
                "scale must have the same number of elements as the features of x, got %lld and %lld",
                (long long)num_elements(scale), (long long)D);
  ATEXN_REQUIRE(num_elements(offset) == D,
                "offset must have the same number of elements as the features of x, got %lld and %lld",
                (long long)num_elements(offset), (long long)D);
  ATEXN_REQUIRE(y->dtype == x->dtype && same_shape(x, y), "y must have the dtype and shape of x");
  ATEXN_REQUIRE(reserve_space_1->rank == 1 && reserve_space_1->dims[0] == N &&
                    reserve_space_2->rank == 1 && reserve_space_2->dims[0] == N,
                "reserve spaces must be rank 1 with %lld elements", (long long)N);
  if (x->device == ATEXN_DEVICE_CPU) {
    return atexn_layer_norm_fwd_cpu(x->dtype, x->data, static_cast<const float*>(scale->data),
                                    static_cast<const float*>(offset->data), N, D, epsilon, y->data,
                                    static_cast<float*>(reserve_space_1->data),
                                    static_cast<float*>(reserve_space_2->data));
  }
  return atexn_layer_norm_fwd(x->dtype, x->data, static_cast<const float*>(scale->data),
                              static_cast<const float*>(offset->data), N, D, epsilon, y->data,
                              static_cast<float*>(reserve_space_1->data),
                              static_cast<float*>(reserve_space_2->data), workspace,
                              workspace_bytes, stream);
}

size_t atexn_fused_layer_norm_grad_workspace_bytes(const atexn_tensor* x, const int* axis,
                                                   int n_axis) {
  int64_t N, D;
  if (!x || atexn_layer_norm_resolve_axes(x->rank, x->dims, axis, n_axis, &N, &D) != ATEXN_OK) return 0;
  if (x->device == ATEXN_DEVICE_CPU) return 0;
  return atexn_layer_norm_bwd_workspace_bytes(x->dtype, N, D);
}

int atexn_fused_layer_norm_grad(const atexn_tensor* y_backprop, const atexn_tensor* x,
                                const atexn_tensor* scale, const atexn_tensor* reserve_space_1,
                                const atexn_tensor* reserve_space_2, const int* axis,
                                int n_axis, atexn_tensor* x_backprop,
                                atexn_tensor* scale_backprop, atexn_tensor* offset_backprop,
                                void* workspace, size_t workspace_bytes, void* stream) {
  ATEXN_TRY(check_tensor(y_backprop, "y_backprop"));
  ATEXN_TRY(check_tensor(x, "x"));
  ATEXN_TRY(check_tensor(scale, "scale"));
  ATEXN_TRY(check_tensor(reserve_space_1, "reserve_space_1"));
  ATEXN_TRY(check_tensor(reserve_space_2, "reserve_space_2"));
  ATEXN_TRY(check_tensor(x_backprop, "x_backprop"));
  ATEXN_TRY(check_tensor(scale_backprop, "scale_backprop"));
  ATEXN_TRY(check_tensor(offset_backprop, "offset_backprop"));
  ATEXN_TRY(check_same_device(x, y_backprop, scale, reserve_space_1, reserve_space_2, x_backprop,
                              scale_backprop, offset_backprop));
  ATEXN_REQUIRE(scale->dtype == ATEXN_F32 && reserve_space_1->dtype == ATEXN_F32 &&
                    reserve_space_2->dtype == ATEXN_F32 && scale_backprop->dtype == ATEXN_F32 &&
                    offset_backprop->dtype == ATEXN_F32,
                "scale, the reserve spaces and the scale/offset gradients must be float32");
  ATEXN_REQUIRE(y_backprop->rank > 0 && x->rank > 0, "input must be at least 1-dimensional");
  ATEXN_REQUIRE(reserve_space_1->rank == 1, "saved mean must be 1-dimensional");
  ATEXN_REQUIRE(reserve_space_2->rank == 1, "saved inverted variance must be 1-dimensional");
  ATEXN_REQUIRE(same_shape(x, y_backprop) && x->dtype == y_backprop->dtype,
                "x and y_backprop must have same shape");
  int64_t N, D;
  ATEXN_TRY(atexn_layer_norm_resolve_axes(x->rank, x->dims, axis, n_axis, &N, &D));
  ATEXN_REQUIRE(num_elements(scale) == D,
                "scale must have the same number of elements as the features of x, got %lld and %lld",
                (long long)num_elements(scale), (long long)D);
  ATEXN_REQUIRE(reserve_space_1->dims[0] == N,
                "reserve_space_1 must have the same number of elements as the batches of x, got %lld and %lld",
                (long long)reserve_space_1->dims[0], (long long)N);
  ATEXN_REQUIRE(reserve_space_2->dims[0] == N,
                "reserve_space_2 must have the same number of elements as the batches of x, got %lld and %lld",
                (long long)reserve_space_2->dims[0], (long long)N);
  ATEXN_REQUIRE(x_backprop->dtype == x->dtype && same_shape(x, x_backprop),
                "x_backprop must have the dtype and shape of x");
  ATEXN_REQUIRE(num_elements(scale_backprop) == D && num_elements(offset_backprop) == D,
                "scale_backprop / offset_backprop must have %lld elements", (long long)D);
  if (x->device == ATEXN_DEVICE_CPU) {
    return atexn_layer_norm_bwd_cpu(x->dtype, y_backprop->data, x->data,
                                    static_cast<const float*>(scale->data),
                                    static_cast<const float*>(reserve_space_1->data),
                                    static_cast<const float*>(reserve_space_2->data), N, D,
                                    x_backprop->data, static_cast<float*>(scale_backprop->data),
                                    static_cast<float*>(offset_backprop->data));
  }
  return atexn_layer_norm_bwd(x->dtype, y_backprop->data, x->data,
                              static_cast<const float*>(scale->data),
                              static_cast<const float*>(reserve_space_1->data),
                              static_cast<const float*>(reserve_space_2->data), N, D,
                              x_backprop->data, static_cast<float*>(scale_backprop->data),
                              static_cast<float*>(offset_backprop->data), workspace,
                              workspace_bytes, stream);
}

size_t atexn_fused_instance_norm_workspace_bytes(const atexn_tensor* x, const char* data_format) {
  int layout;
  int64_t N, C, D;
  if (!x || atexn_instance_norm_resolve_format(x->rank, x->dims, data_format, &layout, &N, &C, &D) != ATEXN_OK) return 0;
  if (x->device == ATEXN_DEVICE_CPU) return 0;
  return atexn_instance_norm_fwd_workspace_bytes(x->dtype, layout, N, C, D);
}

int atexn_fused_instance_norm(const atexn_tensor* x, const atexn_tensor* scale,
                              const atexn_tensor* offset, float epsilon,
                              const char* data_format, atexn_tensor* y,
                              atexn_tensor* reserve_space_1, atexn_tensor* reserve_space_2,
                              void* workspace, size_t workspace_bytes, void* stream) {
  ATEXN_TRY(check_tensor(x, "x"));
  ATEXN_TRY(check_tensor(scale, "scale"));
  ATEXN_TRY(check_tensor(offset, "offset"));
  ATEXN_TRY(check_tensor(y, "y"));
  ATEXN_TRY(check_tensor(reserve_space_1, "reserve_space_1"));
  ATEXN_TRY(check_tensor(reserve_space_2, "reserve_space_2"));
  ATEXN_TRY(check_same_device(x, scale, offset, y, reserve_space_1, reserve_space_2));
  ATEXN_REQUIRE(scale->dtype == ATEXN_F32 && offset->dtype == ATEXN_F32 &&
                    reserve_space_1->dtype == ATEXN_F32 && reserve_space_2->dtype == ATEXN_F32,
                "scale, offset and the reserve spaces must be float32");
  ATEXN_REQUIRE(x->rank > 3, "input must be at least 4-dimensional");
  ATEXN_REQUIRE(scale->rank == 1, "scale must be 1-dimensional");
  ATEXN_REQUIRE(offset->rank == 1, "offset must be 1-dimensional");
  int layout;
  int64_t N, C, D;
  ATEXN_TRY(atexn_instance_norm_resolve_format(x->rank, x->dims, data_format, &layout, &N, &C, &D));
  ATEXN_REQUIRE(scale->dims[0] == C,
                "scale must have the same number of elements as the channels of x, got %lld and %lld",
                (long long)scale->dims[0], (long long)C);
  ATEXN_REQUIRE(offset->dims[0] == C,
                "offset must have the same number of elements as the channels of x, got %lld and %lld",
                (long long)offset->dims[0], (long long)C);
  ATEXN_REQUIRE(y->dtype == x->dtype && same_shape(x, y), "y must have the dtype and shape of x");
  ATEXN_REQUIRE(reserve_space_1->rank == 2 && reserve_space_1->dims[0] == N && reserve_space_1->dims[1] == C &&
                    reserve_space_2->rank == 2 && reserve_space_2->dims[0] == N && reserve_space_2->dims[1] == C,
                "reserve spaces must have shape [%lld, %lld]", (long long)N, (long long)C);
  if (x->device == ATEXN_DEVICE_CPU) {
    return atexn_instance_norm_fwd_cpu(x->dtype, layout, x->data, static_cast<const float*>(scale->data),
                                       static_cast<const float*>(offset->data), N, C, D, epsilon,
                                       y->data, static_cast<float*>(reserve_space_1->data),
                                       static_cast<float*>(reserve_space_2->data));
  }
  return atexn_instance_norm_fwd(x->dtype, layout, x->data, static_cast<const float*>(scale->data),
                                 static_cast<const float*>(offset->data), N, C, D, epsilon, y->data,
                                 static_cast<float*>(reserve_space_1->data),
                                 static_cast<float*>(reserve_space_2->data), workspace,
                                 workspace_bytes, stream);
}

size_t atexn_fused_instance_norm_grad_workspace_bytes(const atexn_tensor* x,
                                                      const char* data_format) {
  int layout;
  int64_t N, C, D;
  if (!x || atexn_instance_norm_resolve_format(x->rank, x->dims, data_format, &layout, &N, &C, &D) != ATEXN_OK) return 0;
  if (x->device == ATEXN_DEVICE_CPU) return 0;
  return atexn_instance_norm_bwd_workspace_bytes(x->dtype, layout, N, C, D);
}

int atexn_fused_instance_norm_grad(const atexn_tensor* y_backprop, const atexn_tensor* x,
                                   const atexn_tensor* scale,
                                   const atexn_tensor* reserve_space_1,
                                   const atexn_tensor* reserve_space_2,
                                   const char* data_format, atexn_tensor* x_backprop,
                                   atexn_tensor* scale_backprop,
                                   atexn_tensor* offset_backprop, void* workspace,
                                   size_t workspace_bytes, void* stream) {
  ATEXN_TRY(check_tensor(y_backprop, "y_backprop"));
  ATEXN_TRY(check_tensor(x, "x"));
  ATEXN_TRY(check_tensor(scale, "scale"));
  ATEXN_TRY(check_tensor(reserve_space_1, "reserve_space_1"));
  ATEXN_TRY(check_tensor(reserve_space_2, "reserve_space_2"));
  ATEXN_TRY(check_tensor(x_backprop, "x_backprop"));
  ATEXN_TRY(check_tensor(scale_backprop, "scale_backprop"));
  ATEXN_TRY(check_tensor(offset_backprop, "offset_backprop"));
  ATEXN_TRY(check_same_device(x, y_backprop, scale, reserve_space_1, reserve_space_2, x_backprop,
                              scale_backprop, offset_backprop));
  ATEXN_REQUIRE(scale->dtype == ATEXN_F32 && reserve_space_1->dtype == ATEXN_F32 &&
                    reserve_space_2->dtype == ATEXN_F32 && scale_backprop->dtype == ATEXN_F32 &&
                    offset_backprop->dtype == ATEXN_F32,
                "scale, the reserve spaces and the scale/offset gradients must be float32");
  ATEXN_REQUIRE(y_backprop->rank > 3, "input must be at least 4-dimensional");
  ATEXN_REQUIRE(scale->rank == 1, "scale must be 1-dimensional");
  ATEXN_REQUIRE(reserve_space_1->rank == 2, "saved mean must be 2-dimensional");
  ATEXN_REQUIRE(reserve_space_2->rank == 2, "saved inverted variance must be 2-dimensional");
  ATEXN_REQUIRE(same_shape(x, y_backprop) && x->dtype == y_backprop->dtype,
                "x and y_backprop must have same shape");
  int layout;
  int64_t N, C, D;
  ATEXN_TRY(atexn_instance_norm_resolve_format(x->rank, x->dims, data_format, &layout, &N, &C, &D));
  ATEXN_REQUIRE(scale->dims[0] == C,
                "scale must have the same number of elements as the channels of x, got %lld and %lld",
                (long long)scale->dims[0], (long long)C);
  ATEXN_REQUIRE(num_elements(reserve_space_1) == N * C,
                "reserve_space_1 must have the same number of elements as the batches*channels of x, got %lld and %lld",
                (long long)num_elements(reserve_space_1), (long long)(N * C));
  ATEXN_REQUIRE(num_elements(reserve_space_2) == N * C,
                "reserve_space_2 must have the same number of elements as the batches*channels of x, got %lld and %lld",
                (long long)num_elements(reserve_space_2), (long long)(N * C));
  ATEXN_REQUIRE(x_backprop->dtype == x->dtype && same_shape(x, x_backprop),
                "x_backprop must have the dtype and shape of x");
  ATEXN_REQUIRE(num_elements(scale_backprop) == C && num_elements(offset_backprop) == C,
                "scale_backprop / offset_backprop must have %lld elements", (long long)C);
  if (x->device == ATEXN_DEVICE_CPU) {
    return atexn_instance_norm_bwd_cpu(x->dtype, layout, y_backprop->data, x->data,
                                       static_cast<const float*>(scale->data),
                                       static_cast<const float*>(reserve_space_1->data),
                                       static_cast<const float*>(reserve_space_2->data), N, C, D,
                                       x_backprop->data, static_cast<float*>(scale_backprop->data),
                                       static_cast<float*>(offset_backprop->data));
  }
  return atexn_instance_norm_bwd(x->dtype, layout, y_backprop->data, x->data,
                                 static_cast<const float*>(scale->data),
                                 static_cast<const float*>(reserve_space_1->data),
                                 static_cast<const float*>(reserve_space_2->data), N, C, D,
                                 x_backprop->data, static_cast<float*>(scale_backprop->data),
                                 static_cast<float*>(offset_backprop->data), workspace,
                                 workspace_bytes, stream);
}

}  // extern "C"
