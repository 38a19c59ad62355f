/* Thin C-ABI launch layer between host C++ and the HIP kernels (gfx950).
 *
 * Plain pointers, sizes and ints only: no HIP, C++ or torch types cross this
 * boundary, so the calculator classes above it (include/sphericart_cuda.hpp)
 * and any foreign-function binding can be built by an ordinary host compiler.
 *
 * Each entry point below names the piece of the reference it stands in for
 * (paths relative to the reference checkout).
 */
#ifndef SPHX_LAUNCH_H
#define SPHX_LAUNCH_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SPHX_EXPORT __attribute__((visibility("default")))

/* Status codes returned by every function of this layer. */
#define SPHX_OK 0
#define SPHX_ERR_ARGUMENT 1    /* null pointer, negative l_max, unknown selector */
#define SPHX_ERR_UNSUPPORTED 2 /* l_max beyond the device tables / LDS capacity */
#define SPHX_ERR_HIP 3         /* a HIP runtime call failed; see sphx_last_error() */

/* What to evaluate next to the values. */
#define SPHX_VALUES 0
#define SPHX_GRADIENTS 1
#define SPHX_HESSIANS 2

/* Largest l_max the constant-memory prefactor tables cover. */
#define SPHX_TABLE_LMAX 64

/* Evaluate real spherical (normalized != 0) or solid (normalized == 0)
 * harmonics up to l_max for n_samples points, enqueued on `stream`.
 *
 *   xyz    device, [n_samples][3]
 *   sph    device, [n_samples][(l_max+1)^2]
 *   dsph   device, [n_samples][3][(l_max+1)^2]     (derivatives >= SPHX_GRADIENTS)
 *   ddsph  device, [n_samples][3][3][(l_max+1)^2]  (derivatives == SPHX_HESSIANS)
 *   stream the hipStream_t value itself (not a pointer to it); NULL = default stream
 *
 * The call returns after enqueueing; it does not synchronise. n_samples == 0
 * returns SPHX_OK before looking at any pointer. The device is taken from the
 * xyz pointer and the caller's current device is restored on return.
 *
 * Replaces sphericart::cuda::spherical_harmonics_cuda_base<T>
 * (sphericart/src/cuda_base.cpp:69-120, declared sphericart/include/cuda_base.hpp)
 * together with the pointer-to-device switch and prefactor upload of
 * SphericalHarmonics<T>::compute_internal (sphericart/src/sphericart_cuda.cpp:115-159).
 */
SPHX_EXPORT int sphx_forward_f32(const float* xyz, size_t n_samples, int l_max, int normalized,
                                 int derivatives, float* sph, float* dsph, float* ddsph,
                                 void* stream);
SPHX_EXPORT int sphx_forward_f64(const double* xyz, size_t n_samples, int l_max, int normalized,
                                 int derivatives, double* sph, double* dsph, double* ddsph,
                                 void* stream);

/* Vector-Jacobian product of the forward pass for reverse-mode callers:
 *
 *   xyz_grad[i][a] (+)= sum_k dsph[i][a][k] * sph_grad[i][k]
 *
 *   dsph      device, [n_samples][3][n_total]   (as written by sphx_forward_*)
 *   sph_grad  device, [n_samples][n_total]      gradient of the caller's scalar w.r.t. sph
 *   xyz_grad  device, [n_samples][3]
 *   n_total   row length, (l_max+1)^2
 *   accumulate  0: overwrite xyz_grad; otherwise add to what it holds
 *
 * Enqueued on `stream` like the forward pass; n_samples == 0 returns SPHX_OK.
 * Replaces spherical_harmonics_backward_cuda_base<T>
 * (sphericart/src/cuda_base.cpp:156-183) and its backward_kernel
 * (sphericart/src/sphericart_impl.cu:650-684); same arguments plus `accumulate`. */
SPHX_EXPORT int sphx_backward_f32(const float* dsph, const float* sph_grad, size_t n_samples,
                                  int n_total, float* xyz_grad, int accumulate, void* stream);
SPHX_EXPORT int sphx_backward_f64(const double* dsph, const double* sph_grad, size_t n_samples,
                                  int n_total, double* xyz_grad, int accumulate, void* stream);

/* The same one order up, for callers that differentiate through the gradients:
 *
 *   xyz_grad[i][b] (+)= sum_a sum_k ddsph[i][a][b][k] * dsph_grad[i][a][k]
 *
 *   ddsph      device, [n_samples][3][3][n_total]
 *   dsph_grad  device, [n_samples][3][n_total]   gradient of the caller's scalar w.r.t. dsph
 *
 * The reference has no kernel for this; its torch binding evaluates it as
 * torch.sum(grad.unsqueeze(2) * ddsph, dim=(1, 3))
 * (sphericart-torch/python/sphericart/torch/register.py:106-110). */
SPHX_EXPORT int sphx_backward_second_f32(const float* ddsph, const float* dsph_grad,
                                         size_t n_samples, int n_total, float* xyz_grad,
                                         int accumulate, void* stream);
SPHX_EXPORT int sphx_backward_second_f64(const double* ddsph, const double* dsph_grad,
                                         size_t n_samples, int n_total, double* xyz_grad,
                                         int accumulate, void* stream);

/* Forward and backward pass fused, for callers that only need the gradient of a
 * scalar with respect to the coordinates (training):
 *
 *   xyz_grad[i][a] (+)= sum_k (d sph[i][k] / d xyz[i][a]) * sph_grad[i][k]
 *
 * without dsph ever reaching memory: reads xyz and sph_grad, writes xyz_grad.
 * For l_max <= 6 the sum runs over k in index order, one rounding per
 * operation: the numbers are those of sphx_forward_* followed by a sequential
 * contraction. Beyond that the terms are added in another order (lanes, then a
 * butterfly), so the result agrees with that combination to rounding only.
 * No counterpart in the reference, whose torch binding recomputes dsph in
 * memory for its backward pass
 * (sphericart-torch/python/sphericart/torch/register.py:96-103). */
SPHX_EXPORT int sphx_vjp_f32(const float* xyz, const float* sph_grad, size_t n_samples, int l_max,
                             int normalized, float* xyz_grad, int accumulate, void* stream);
SPHX_EXPORT int sphx_vjp_f64(const double* xyz, const double* sph_grad, size_t n_samples, int l_max,
                             int normalized, double* xyz_grad, int accumulate, void* stream);

/* float32 arrays, evaluated in float64 and rounded once: what sphx_forward_f64
 * returns for the same points, converted to float (round to nearest even).
 * For callers that need float32 storage beyond the range of float32
 * arithmetic: evaluated in float, the prefactors and Q_l^l = (2l-1)!! of
 * sphericart/include/templates.hpp:54-97 overflow from l = 29 (the outputs of
 * the reference and of sphx_forward_f32 hold NaN and inf there) and underflow
 * to exact zeros at high |m| from l of about 20. No counterpart in the
 * reference; never chosen implicitly, since parity with the reference is
 * defined on sphx_forward_f32.
 *
 * Beyond the closed forms (l_max > 6; l_max > 1 with second derivatives) this
 * is one launch of the recursion kernel in its mixed variant: it reads the
 * float coordinates, keeps tables and iterates in float64 and stages float
 * rows, each number rounded as it is stored. No workspace is read or written
 * then, and nothing is allocated. At or below the closed forms, and where one
 * point's float rows and float64 tables exceed a CU's LDS, the points are
 * widened, evaluated into float64 rows in a workspace and narrowed:
 *
 *   workspace        device memory, 16-byte aligned, of workspace_bytes bytes;
 *                    the points are processed in chunks of as many as it holds
 *                    (8 * (3 + (l_max+1)^2 * {1, 4, 13}) bytes each), enqueued
 *                    one after the other on `stream`. NULL: the call takes a
 *                    workspace of at most 256 MiB from the device's memory
 *                    pool and returns it, both in stream order
 *                    (hipMallocAsync / hipFreeAsync): it still only enqueues.
 *
 * sphx_forward_f32_via_f64_workspace returns the size with which n_samples
 * points are one chunk (0 for invalid arguments). */
SPHX_EXPORT int sphx_forward_f32_via_f64(const float* xyz, size_t n_samples, int l_max,
                                         int normalized, int derivatives, float* sph, float* dsph,
                                         float* ddsph, void* workspace, size_t workspace_bytes,
                                         void* stream);
SPHX_EXPORT size_t sphx_forward_f32_via_f64_workspace(size_t n_samples, int l_max, int derivatives);

/* sphx_forward_f32_via_f64 for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. No counterpart in the reference. The call allocates and frees
 * nothing and only enqueues on `stream`. Beyond the closed forms (l_max > 6,
 * or > 1 with second derivatives) it is the one launch of the kernel that
 * computes in float64 and stores float rows, as in sphx_forward_f32_via_f64:
 * no workspace is needed and any number of points goes. Up to there the
 * float64 rows are staged in a scratch array of 32 MiB that is part of the
 * library's device code (every GPU the library runs on holds its own copy
 * until the process ends), and the whole call must fit into it: more than
 * sphx_forward_f32_via_f64_static_capacity(l_max, derivatives) points
 * (32 MiB / (8 * (3 + (l_max+1)^2 * {1, 4, 13})); 0 for invalid arguments)
 * return SPHX_ERR_UNSUPPORTED with a message that names the limit; larger
 * batches are passed in slices. All calls on one GPU share that GPU's array:
 * calls that overlap in time on one GPU (two streams, two threads) race and
 * must be ordered by the caller. Same results as sphx_forward_f32_via_f64. */
SPHX_EXPORT int sphx_forward_f32_via_f64_static(const float* xyz, size_t n_samples, int l_max,
                                                int normalized, int derivatives, float* sph,
                                                float* dsph, float* ddsph, void* stream);
SPHX_EXPORT size_t sphx_forward_f32_via_f64_static_capacity(int l_max, int derivatives);

/* Host copy of the prefactor table the kernels use for this l_max: the F_l^m
 * block followed by the Q_l^m-recursion block, (l_max+1)(l_max+2) numbers.
 * Replaces compute_sph_prefactors<T> (sphericart/include/templates.hpp:54-97)
 * as called from the device class (sphericart/src/sphericart_cuda.cpp:57). */
SPHX_EXPORT int sphx_prefactors_f32(int l_max, float* out);
SPHX_EXPORT int sphx_prefactors_f64(int l_max, double* out);

/* Number of visible GPUs, or a negative value when the HIP runtime reports an
 * error. Replaces the cudaGetDeviceCount probe of the device-class constructor
 * (sphericart/src/sphericart_cuda.cpp:54). */
SPHX_EXPORT int sphx_device_count(void);

/* Message of the last failure on the calling thread ("" if none). No
 * counterpart in the reference, which throws from inside its launcher
 * (sphericart/src/cuda_base.cpp:75-84); the classes above this layer turn the
 * message into the same std::runtime_error. */
SPHX_EXPORT const char* sphx_last_error(void);

/* Yardsticks for benchmarks; none of them has a counterpart in the reference and none is on the path of an
 * evaluation. sphx_probe_empty_launch enqueues a kernel that does nothing (what a launch costs whatever it
 * computes); sphx_probe_fill writes `bytes` bytes (a multiple of 16, `out` aligned to 16) with the store pattern
 * of the evaluator's flush and nothing to compute (how fast plain stores fill HBM); sphx_probe_host_cost_f64
 * makes `calls` calls in a row without waiting for the GPU, values and gradients of normalised harmonics in
 * float64, through sphx_forward_f64 (`through` = 0) or through a calculator of the sphericart_cuda_* C API
 * (1), and reports the host seconds per call. */
SPHX_EXPORT int sphx_probe_empty_launch(void* stream);
SPHX_EXPORT int sphx_probe_fill(void* out, size_t bytes, void* stream);
SPHX_EXPORT int sphx_probe_host_cost_f64(int through, const double* xyz, size_t n_samples, int l_max, double* sph,
                                         double* dsph, void* stream, int calls, double* seconds_per_call);

/* Launch geometry chosen for a call of this shape (for benchmarks and tests):
 * samples per workgroup tile, threads per workgroup, LDS bytes per workgroup,
 * number of workgroups. Returns a status code. No counterpart in the reference
 * (its geometry is fixed at 8 x 8 threads, sphericart/src/cuda_base.cpp:89-94). */
SPHX_EXPORT int sphx_plan(size_t n_samples, int l_max, int derivatives, int is_f64,
                          int* tile_samples, int* threads, int* lds_bytes, int* workgroups);

/* The same as text: the kernel or kernels a call of this shape launches, with
 * their template arguments as a profiler prints them, and the geometry of each
 * launch. At most `capacity` bytes are written, NUL included. For benchmark
 * records; no counterpart in the reference. */
SPHX_EXPORT int sphx_describe_plan(size_t n_samples, int l_max, int derivatives, int is_f64,
                                   int normalized, char* out, size_t capacity);

/* Override one decision of the launch planner, for measurements and for tests
 * that want both sides of a choice exercised: `name` is one of the SPHX_*
 * names listed in sphx_plan.hpp (SPHX_TILE, SPHX_JOB_LIST, ...), unknown
 * names return SPHX_ERR_ARGUMENT. Process-wide; takes effect with the next
 * call on any thread. sphx_reset_switches() drops all overrides. Without
 * overrides a call is planned from its shape alone. The environment variables
 * of the same names are read once, when the library is first used, and only if
 * SPHX_DEBUG_SWITCHES is set. No counterpart in the reference. */
SPHX_EXPORT int sphx_set_switch(const char* name, int value);
SPHX_EXPORT void sphx_reset_switches(void);

#ifdef __cplusplus
}
#endif

#endif
