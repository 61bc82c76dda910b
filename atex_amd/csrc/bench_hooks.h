/* Entry points that exist only in the benchmark build of the library
 * (libatex_norms_hip_bench.so: the product sources compiled with -DATEXN_BENCH_BUILD).  The
 * product library exports none of them and keeps no process-wide state; bench.py and the tests
 * that force a particular kernel family load the benchmark build for these. */
#ifndef ATEXN_BENCH_HOOKS_H_
#define ATEXN_BENCH_HOOKS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Sets one launch-planning parameter (struct Tuning in plan.h lists the names) for the whole
 * process.  A *_workspace_bytes query and the call it sizes must run under the same settings.
 * "bwd_stage_mask" (1: only the row kernel of a backward call, 2: only its column reduction,
 * 3: both) is the one parameter whose non-default values give incomplete results. */
int atexn_set_tuning(const char* name, int value);

/* Text description of the kernels a backward call of the given shape launches and whether
 * bwd_stage_mask can time its row kernel alone ("...; alone=1"). */
int atexn_bench_describe_bwd(int op, int dtype, int layout, int64_t N, int64_t C, int64_t D,
                             char* out, size_t out_bytes);

/* Writes the current device's record of "the last call whose workgroups waited for each other in
 * vain": recent != 0 makes it this moment (the exchange kernels of the next 256 calls give a wait
 * up after a few polls), recent == 0 makes it long ago (patient waits).  Synchronous. */
int atexn_bench_mark_exchange_trouble(int recent);

/* How many exchange-kernel calls ago that record was last written by a kernel (or by the function
 * above), saturated at INT_MAX; -1 when it cannot be read.  Synchronises the device. */
int atexn_bench_exchange_trouble_age(void);

/* Launches, on `stream`, a kernel that does nothing but hold `workgroups` whole compute units
 * (1024 threads and 158 of the CU's 160 KB of LDS each) for about `milliseconds` (at most 100): what a large kernel
 * of another library does to the exchange kernels when it runs beside them on the same GPU.
 * Every wave leaves when the time is up, or after a fixed number of loop passes whatever the
 * clock says.  For the tests and measurements of that situation. */
int atexn_bench_occupy(int workgroups, double milliseconds, void* stream);

#ifdef __cplusplus
}
#endif
#endif
