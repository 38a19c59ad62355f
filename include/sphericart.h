/* C API of the MI355X (gfx950, HIP) evaluator: the device half of the
 * reference's C API, with the same symbol names, argument lists and ownership
 * rules, so that a foreign-function binding written against the reference
 * (for instance python/src/sphericart/_c_lib.py:240-400) loads this library
 * unchanged.
 *
 * Reference: declarations sphericart/include/sphericart.h:91-104 (opaque
 * calculator types) and :641-779 (the twenty sphericart_cuda_* functions);
 * definitions sphericart/src/sphericart-capi.cpp:637-876.
 *
 * Conventions (all as in the reference):
 *  - `*_new` returns a calculator owned by the caller, to be released with the
 *    matching `*_delete`; it returns NULL when the calculator cannot be built
 *    (no usable GPU, l_max not supported).
 *  - every array is device memory allocated by the caller, contiguous and
 *    row-major; `cuda_stream` is the native stream handle by value
 *    (a hipStream_t), NULL for the default stream; calls do not synchronise.
 *  - on failure a compute function prints `fatal error: <reason>` on stdout
 *    and calls abort().
 *
 * The reference's host (CPU) entry points, sphericart_spherical_harmonics_* and
 * sphericart_solid_harmonics_*, are not part of this library.
 */
#ifndef SPHERICART_H
#define SPHERICART_H

#include <stddef.h>

#ifndef SPHERICART_EXPORT
#define SPHERICART_EXPORT __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
#include "sphericart_cuda.hpp"

using sphericart_cuda_spherical_harmonics_calculator_t = sphericart::cuda::SphericalHarmonics<double>;
using sphericart_cuda_spherical_harmonics_calculator_f_t = sphericart::cuda::SphericalHarmonics<float>;
using sphericart_cuda_solid_harmonics_calculator_t = sphericart::cuda::SolidHarmonics<double>;
using sphericart_cuda_solid_harmonics_calculator_f_t = sphericart::cuda::SolidHarmonics<float>;

extern "C" {
#else
typedef struct sphericart_cuda_spherical_harmonics_calculator_t
    sphericart_cuda_spherical_harmonics_calculator_t;
typedef struct sphericart_cuda_spherical_harmonics_calculator_f_t
    sphericart_cuda_spherical_harmonics_calculator_f_t;
typedef struct sphericart_cuda_solid_harmonics_calculator_t sphericart_cuda_solid_harmonics_calculator_t;
typedef struct sphericart_cuda_solid_harmonics_calculator_f_t
    sphericart_cuda_solid_harmonics_calculator_f_t;
#endif

/* ---- spherical harmonics, double (reference sphericart.h:641-689) ---- */

SPHERICART_EXPORT sphericart_cuda_spherical_harmonics_calculator_t*
sphericart_cuda_spherical_harmonics_new(size_t l_max);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_delete(
    sphericart_cuda_spherical_harmonics_calculator_t* calculator);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array(
    sphericart_cuda_spherical_harmonics_calculator_t* calculator, const double* xyz,
    size_t n_samples, double* sph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array_with_gradients(
    sphericart_cuda_spherical_harmonics_calculator_t* calculator, const double* xyz,
    size_t n_samples, double* sph, double* dsph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array_with_hessians(
    sphericart_cuda_spherical_harmonics_calculator_t* calculator, const double* xyz,
    size_t n_samples, double* sph, double* dsph, double* ddsph, void* cuda_stream);

/* ---- spherical harmonics, float (reference sphericart.h:645-708) ---- */

SPHERICART_EXPORT sphericart_cuda_spherical_harmonics_calculator_f_t*
sphericart_cuda_spherical_harmonics_new_f(size_t l_max);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_delete_f(
    sphericart_cuda_spherical_harmonics_calculator_f_t* calculator);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array_f(
    sphericart_cuda_spherical_harmonics_calculator_f_t* calculator, const float* xyz,
    size_t n_samples, float* sph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array_with_gradients_f(
    sphericart_cuda_spherical_harmonics_calculator_f_t* calculator, const float* xyz,
    size_t n_samples, float* sph, float* dsph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_spherical_harmonics_compute_array_with_hessians_f(
    sphericart_cuda_spherical_harmonics_calculator_f_t* calculator, const float* xyz,
    size_t n_samples, float* sph, float* dsph, float* ddsph, void* cuda_stream);

/* ---- solid harmonics, double (reference sphericart.h:710-758) ---- */

SPHERICART_EXPORT sphericart_cuda_solid_harmonics_calculator_t* sphericart_cuda_solid_harmonics_new(
    size_t l_max);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_delete(
    sphericart_cuda_solid_harmonics_calculator_t* calculator);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array(
    sphericart_cuda_solid_harmonics_calculator_t* calculator, const double* xyz, size_t n_samples,
    double* sph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array_with_gradients(
    sphericart_cuda_solid_harmonics_calculator_t* calculator, const double* xyz, size_t n_samples,
    double* sph, double* dsph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array_with_hessians(
    sphericart_cuda_solid_harmonics_calculator_t* calculator, const double* xyz, size_t n_samples,
    double* sph, double* dsph, double* ddsph, void* cuda_stream);

/* ---- solid harmonics, float (reference sphericart.h:714-779) ---- */

SPHERICART_EXPORT sphericart_cuda_solid_harmonics_calculator_f_t*
sphericart_cuda_solid_harmonics_new_f(size_t l_max);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_delete_f(
    sphericart_cuda_solid_harmonics_calculator_f_t* calculator);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array_f(
    sphericart_cuda_solid_harmonics_calculator_f_t* calculator, const float* xyz, size_t n_samples,
    float* sph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array_with_gradients_f(
    sphericart_cuda_solid_harmonics_calculator_f_t* calculator, const float* xyz, size_t n_samples,
    float* sph, float* dsph, void* cuda_stream);

SPHERICART_EXPORT void sphericart_cuda_solid_harmonics_compute_array_with_hessians_f(
    sphericart_cuda_solid_harmonics_calculator_f_t* calculator, const float* xyz, size_t n_samples,
    float* sph, float* dsph, float* ddsph, void* cuda_stream);

#ifdef __cplusplus
}
#endif

#endif
