/*
 * atex_norms.h -- C ABI of libatex_norms_hip.so: fused LayerNorm / InstanceNorm forward
 * and backward on AMD MI355X (gfx950), the drop-in for the device side of NVIDIA/atex's
 * nv_norms custom ops.
 *
 * The same ops also have host (CPU) kernels, as the reference registers CPU kernels beside its
 * GPU ones: atexn_*_cpu at the kernel level, and the op level picks them when the tensor
 * descriptors say ATEXN_DEVICE_CPU.
 *
 * Two levels:
 *   1. kernel level (atexn_layer_norm_fwd ...): flat [N, D] / [N, C, D] / [N, D, C] views,
 *      raw device pointers, caller-owned workspace, a HIP stream.  These replace the
 *      reference's GPU functors functor::FusedLayerNorm<GPUDevice,T,U> etc.
 *   2. op level (atexn_fused_layer_norm ...): shaped tensor descriptors plus the op's
 *      attributes; performs the validation, axis packing and flattening that the
 *      reference's OpKernel::Compute methods perform, then calls level 1.  A TensorFlow
 *      OpKernel (or any other host) allocates the outputs and calls these.
 *
 * Conventions
 *   - every pointer that is read or written by a kernel is a DEVICE pointer;
 *   - x / y / dy / dx use the storage dtype; gamma, beta, the saved statistics, dgamma and
 *     dbeta are always float32;
 *   - the saved statistics are the mean and the INVERSE STANDARD DEVIATION
 *     rsqrt(biased_variance + epsilon) (reference: cc/kernels/norm_util.h:253-258);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream); every call is
 *     asynchronous on it, re-entrant, allocates nothing and keeps no device state that a
 *     result depends on (atexn_layer_norm_bwd_static is the one exception, see there; besides,
 *     one 4-byte word per device remembers the last call whose workgroups waited for each other
 *     in vain, and only makes the next calls give such waits up sooner); the library has no
 *     process-wide settings: launch plans depend on the sizes and the device alone.  One
 *     environment variable is read, once, at the first call: ATEXN_NO_EXCHANGE=1 keeps every
 *     InstanceNorm call on kernels that need no group of workgroups resident on the GPU
 *     together (two launches per direction instead of one for some shapes; same results up to
 *     the order of a few float32 additions in the statistics, same workspace sizes) -- for
 *     processes that keep other kernels running on more than half of the GPU's compute units
 *     all the time, under which the one-launch kernels are correct but two to three times slower
 *     than the two launches;
 *   - the device the stream belongs to must be the calling thread's current device: launch
 *     plans and workspace sizes are made for the current device's compute-unit count;
 *   - data pointers need only the alignment of their element type (2 or 4 bytes): the
 *     kernels' 16-byte accesses work at any element offset, so slices of larger tensors
 *     can be passed as they are;
 *   - `workspace` is device scratch of at least *_workspace_bytes(...) bytes, 256-byte
 *     aligned; it may be NULL when that size is 0;
 *   - return value: ATEXN_OK, ATEXN_INVALID_ARGUMENT (nothing launched) or
 *     ATEXN_LAUNCH_ERROR (a HIP call failed); atexn_last_error() gives the detail of the
 *     calling thread's last failure.  Nothing aborts or throws across this boundary
 *     (the reference aborts on a launch failure, norm_util.h:77);
 *   - empty inputs (N * D == 0 or N * C * D == 0) succeed without reading or writing anything
 *     (mean / inv_std stay unwritten even when N > 0, as in the reference, whose functors
 *     return at once on an empty x, fused_layer_norm_op.cu:811-813); the
 *     backward entry points then zero-fill dgamma / dbeta, as the reference's CPU functor
 *     does (fused_layer_norm_op.cc:96-103) -- its GPU functor leaves them unwritten
 *     (fused_layer_norm_op.cu:904-906).
 */
#ifndef ATEX_NORMS_H_
#define ATEX_NORMS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage dtype of x / y / dy / dx.  The reference registers T in {half, float}
 * (cc/ops/norm_ops.cc:155-156); bfloat16 is an extension. */
enum { ATEXN_F32 = 0, ATEXN_F16 = 1, ATEXN_BF16 = 2 };

/* InstanceNorm memory layout after flattening the spatial dims to D
 * (fused_instance_norm_op.cc:363-373): channel-first [N, C, D] or channels-last [N, D, C]. */
enum { ATEXN_LAYOUT_NC_ = 0, ATEXN_LAYOUT_N_C = 1 };

enum { ATEXN_OK = 0, ATEXN_INVALID_ARGUMENT = 1, ATEXN_LAUNCH_ERROR = 2 };

/* Where a tensor's memory lives (op level).  The zero value is the GPU. */
enum { ATEXN_DEVICE_GPU = 0, ATEXN_DEVICE_CPU = 1 };

#define ATEXN_MAX_RANK 8

const char* atexn_status_string(int status);
/* Message of the calling thread's most recent non-OK return ("" if none). */
const char* atexn_last_error(void);
/* ABI version of this header: bumps when a signature changes. */
int atexn_abi_version(void);

/* ------------------------------------------------------------------ kernel level */

/* Replaces functor::FusedLayerNorm<GPUDevice,T,U>::operator()
 * (cc/kernels/fused_layer_norm_op.cu:805-893), whose scratch came from
 * context->allocate_temp (:853-867). y may alias x. */
size_t atexn_layer_norm_fwd_workspace_bytes(int dtype, int64_t N, int64_t D);
int atexn_layer_norm_fwd(int dtype, const void* x, const float* gamma, const float* beta,
                         int64_t N, int64_t D, float epsilon, void* y, float* mean,
                         float* inv_std, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Replaces functor::FusedLayerNormGrad<GPUDevice,T,U>::operator()
 * (cc/kernels/fused_layer_norm_op.cu:895-1030). dx may alias dy (in-place gradient), not x. */
size_t atexn_layer_norm_bwd_workspace_bytes(int dtype, int64_t N, int64_t D);
int atexn_layer_norm_bwd(int dtype, const void* dy, const void* x, const float* gamma,
                         const float* mean, const float* inv_std, int64_t N, int64_t D,
                         void* dx, float* dgamma, float* dbeta, void* workspace,
                         size_t workspace_bytes, void* stream);

/* atexn_layer_norm_bwd without a workspace argument, for callers that cannot allocate device
 * memory at the point of the call (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference, whose functor allocates its
 * scratch through the framework.  The scratch is a static device array of
 * ATEXN_STATIC_SCRATCH_BYTES inside the library (every GPU the library runs on holds it from
 * module load to process exit); the call allocates and frees nothing.  Problems whose
 * atexn_layer_norm_bwd_workspace_bytes exceeds that size are rejected with
 * ATEXN_INVALID_ARGUMENT.  All calls on one GPU share the one array: calls that overlap in
 * time on the same GPU (two streams, two threads) race; serialise them or use
 * atexn_layer_norm_bwd with separate workspaces.  Nothing has to be cleared between calls
 * (the kernels write every scratch word before they read it).  The first call on a device
 * looks the array's address up (hipGetSymbolAddress); make that call outside stream capture.
 * Results are bit-identical to atexn_layer_norm_bwd. */
#define ATEXN_STATIC_SCRATCH_BYTES (8u << 20)
int atexn_layer_norm_bwd_static(int dtype, const void* dy, const void* x, const float* gamma,
                                const float* mean, const float* inv_std, int64_t N, int64_t D,
                                void* dx, float* dgamma, float* dbeta, void* stream);

/* Replaces functor::FusedInstanceNorm<GPUDevice,T,U>::operator()
 * (cc/kernels/fused_instance_norm_op.cu:1458-1517). mean / inv_std are [N, C] in both
 * layouts. y may alias x.  Size limits (ATEXN_INVALID_ARGUMENT beyond them): N and C below 2^31;
 * channels-last also N below 2^24 and C at most 65535 * 2048. */
size_t atexn_instance_norm_fwd_workspace_bytes(int dtype, int layout, int64_t N, int64_t C,
                                               int64_t D);
int atexn_instance_norm_fwd(int dtype, int layout, const void* x, const float* gamma,
                            const float* beta, int64_t N, int64_t C, int64_t D,
                            float epsilon, void* y, float* mean, float* inv_std,
                            void* workspace, size_t workspace_bytes, void* stream);

/* Replaces functor::FusedInstanceNormGrad<GPUDevice,T,U>::operator()
 * (cc/kernels/fused_instance_norm_op.cu:1519-1561). dgamma / dbeta are [C]; dx may alias dy,
 * not x. */
size_t atexn_instance_norm_bwd_workspace_bytes(int dtype, int layout, int64_t N, int64_t C,
                                               int64_t D);
int atexn_instance_norm_bwd(int dtype, int layout, const void* dy, const void* x,
                            const float* gamma, const float* mean, const float* inv_std,
                            int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
                            float* dbeta, void* workspace, size_t workspace_bytes,
                            void* stream);

/* ------------------------------------------------------------- kernel level, host memory */

/* The CPU kernels of the four ops: counterparts of functor::FusedLayerNorm<CPUDevice,T,U>,
 * FusedLayerNormGrad<CPUDevice,T,U> (cc/kernels/fused_layer_norm_op.cc:27-223, registered
 * :465-478) and FusedInstanceNorm[Grad]<CPUDevice,T,U> (cc/kernels/fused_instance_norm_op.cc:
 * 39-284, registered :541-554).  Every pointer is a HOST pointer; the calls are synchronous,
 * need no workspace and no GPU, and use up to ATEXN_CPU_THREADS (environment; default: all)
 * host threads.  Same arguments, aliasing rules, return codes and empty-input behaviour as
 * the GPU entry points (an empty backward zero-fills dgamma / dbeta, fused_layer_norm_op.cc:
 * 96-103).  Results do not depend on the number of threads. */
int atexn_layer_norm_fwd_cpu(int dtype, const void* x, const float* gamma, const float* beta,
                             int64_t N, int64_t D, float epsilon, void* y, float* mean,
                             float* inv_std);
int atexn_layer_norm_bwd_cpu(int dtype, const void* dy, const void* x, const float* gamma,
                             const float* mean, const float* inv_std, int64_t N, int64_t D,
                             void* dx, float* dgamma, float* dbeta);
int atexn_instance_norm_fwd_cpu(int dtype, int layout, const void* x, const float* gamma,
                                const float* beta, int64_t N, int64_t C, int64_t D,
                                float epsilon, void* y, float* mean, float* inv_std);
int atexn_instance_norm_bwd_cpu(int dtype, int layout, const void* dy, const void* x,
                                const float* gamma, const float* mean, const float* inv_std,
                                int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
                                float* dbeta);

/* ---------------------------------------------------------------------- op level */

/* A dense row-major tensor as the op sees it. `dtype` is ATEXN_F32/F16/BF16, `device` is
 * ATEXN_DEVICE_GPU (data is a device pointer) or ATEXN_DEVICE_CPU (data is a host pointer).
 * All tensors of one call must be on the same device: the op then runs the GPU kernels on
 * `stream`, or the CPU kernels synchronously (workspace and stream are ignored, the workspace
 * queries return 0), the way a framework picks a registered kernel by device placement. */
typedef struct atexn_tensor {
  int dtype;
  int rank;
  int64_t dims[ATEXN_MAX_RANK];
  void* data; /* may be NULL only if the tensor has no elements */
  int device;
} atexn_tensor;

/* Axis handling of FusedLayerNorm (cc/ops/norm_ops.cc:18-52,
 * cc/kernels/fused_layer_norm_op.cc:252-282): negative axes wrap, the set is sorted and
 * de-duplicated and must be packed up to the last dim; N = product of the leading dims,
 * D = product of the normalised dims.  Pure host code. */
int atexn_layer_norm_resolve_axes(int rank, const int64_t* dims, const int* axis, int n_axis,
                                  int64_t* N, int64_t* D);

/* data_format handling of FusedInstanceNorm (cc/kernels/fused_instance_norm_op.cc:25-34,
 * :343-373): accepted iff len > 2, [0] == 'N' and ([1] == 'C' or [last] == 'C'); a 'C' in
 * position 1 means channel-first.  data_format == NULL means the op default "N...C".
 * Requires rank >= 4.  Pure host code. */
int atexn_instance_norm_resolve_format(int rank, const int64_t* dims, const char* data_format,
                                       int* layout, int64_t* N, int64_t* C, int64_t* D);

/* FusedLayerNorm (cc/ops/norm_ops.cc:148-159; Compute: fused_layer_norm_op.cc:295-352).
 * y: same shape as x; mean, inv_std: rank 1 with N elements. */
size_t atexn_fused_layer_norm_workspace_bytes(const atexn_tensor* x, const int* axis,
                                              int n_axis);
int atexn_fused_layer_norm(const atexn_tensor* x, const atexn_tensor* scale,
                           const atexn_tensor* offset, float epsilon, const int* axis,
                           int n_axis, atexn_tensor* y, atexn_tensor* reserve_space_1,
                           atexn_tensor* reserve_space_2, void* workspace,
                           size_t workspace_bytes, void* stream);

/* FusedLayerNormGrad (cc/ops/norm_ops.cc:161-174; Compute: fused_layer_norm_op.cc:370-458).
 * scale_backprop / offset_backprop hold D elements (any shape). */
size_t atexn_fused_layer_norm_grad_workspace_bytes(const atexn_tensor* x, const int* axis,
                                                   int n_axis);
int atexn_fused_layer_norm_grad(const atexn_tensor* y_backprop, const atexn_tensor* x,
                                const atexn_tensor* scale, const atexn_tensor* reserve_space_1,
                                const atexn_tensor* reserve_space_2, const int* axis,
                                int n_axis, atexn_tensor* x_backprop,
                                atexn_tensor* scale_backprop, atexn_tensor* offset_backprop,
                                void* workspace, size_t workspace_bytes, void* stream);

/* FusedInstanceNorm (cc/ops/norm_ops.cc:176-187; Compute: fused_instance_norm_op.cc:328-406).
 * mean, inv_std: rank 2, [N, C]. */
size_t atexn_fused_instance_norm_workspace_bytes(const atexn_tensor* x,
                                                 const char* data_format);
int atexn_fused_instance_norm(const atexn_tensor* x, const atexn_tensor* scale,
                              const atexn_tensor* offset, float epsilon,
                              const char* data_format, atexn_tensor* y,
                              atexn_tensor* reserve_space_1, atexn_tensor* reserve_space_2,
                              void* workspace, size_t workspace_bytes, void* stream);

/* FusedInstanceNormGrad (cc/ops/norm_ops.cc:189-202; Compute:
 * fused_instance_norm_op.cc:430-534). */
size_t atexn_fused_instance_norm_grad_workspace_bytes(const atexn_tensor* x,
                                                      const char* data_format);
int atexn_fused_instance_norm_grad(const atexn_tensor* y_backprop, const atexn_tensor* x,
                                   const atexn_tensor* scale,
                                   const atexn_tensor* reserve_space_1,
                                   const atexn_tensor* reserve_space_2,
                                   const char* data_format, atexn_tensor* x_backprop,
                                   atexn_tensor* scale_backprop,
                                   atexn_tensor* offset_backprop, void* workspace,
                                   size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* ATEX_NORMS_H_ */
