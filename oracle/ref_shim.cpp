// TEST INFRASTRUCTURE ONLY. Thin extern "C" driver around the *reference*
// CPU classes, compiled together with the reference's own sphericart.cpp
// (from where it lies, outside this repository) into oracle/_ref/.
//
// Nothing here restates any arithmetic: every number comes out of
//   sphericart::SphericalHarmonics<T> / sphericart::SolidHarmonics<T>
//     (sphericart/include/sphericart.hpp, sphericart/src/sphericart.cpp:25-476)
//   compute_sph_prefactors<T>            (sphericart/include/templates.hpp:54-97)
//   generic_sph<T, ..., HARDCODED_LMAX=1> (sphericart/include/templates.hpp:617-710)
//
// The entry points mirror oracle/sphx_oracle.cpp one for one so that a test
// can swap the two libraries.

#define _SPHERICART_INTERNAL_IMPLEMENTATION
#include "sphericart.hpp"

#include <cstddef>
#include <cstdio>
#include <exception>
#include <vector>

namespace {

template <typename T>
int run(const T* xyz, size_t n, int l_max, int normalized, int mode, T* sph, T* dsph, T* ddsph) {
    try {
        const size_t ny = static_cast<size_t>(l_max + 1) * (l_max + 1);
        auto go = [&](auto& calc) {
            if (mode == 0) {
                calc.compute_array(xyz, 3 * n, sph, n * ny);
            } else if (mode == 1) {
                calc.compute_array_with_gradients(xyz, 3 * n, sph, n * ny, dsph, 3 * n * ny);
            } else {
                calc.compute_array_with_hessians(
                    xyz, 3 * n, sph, n * ny, dsph, 3 * n * ny, ddsph, 9 * n * ny
                );
            }
        };
        if (normalized) {
            sphericart::SphericalHarmonics<T> calc(static_cast<size_t>(l_max));
            go(calc);
        } else {
            sphericart::SolidHarmonics<T> calc(static_cast<size_t>(l_max));
            go(calc);
        }
    } catch (const std::exception& e) {
        std::fprintf(stderr, "sphx_ref: %s\n", e.what());
        return 1;
    }
    return 0;
}

// Recursion route with only l <= 1 hardcoded and no Hessians: the route the
// reference's own test_hardcoding.cpp:21-33 compares the hardcoded one with.
template <typename T>
int run_recursion_route(const T* xyz, size_t n, int l_max, int normalized, int mode, T* sph, T* dsph) {
    if (l_max < 2 || mode > 1) {
        return 2;
    }
    const size_t nq = static_cast<size_t>(l_max + 1) * (l_max + 2) / 2;
    std::vector<T> pref(2 * nq);
    std::vector<T> buffers(3 * nq * static_cast<size_t>(omp_get_max_threads()));
    compute_sph_prefactors<T>(l_max, pref.data());
    if (normalized) {
        if (mode == 0) {
            generic_sph<T, false, false, true, 1>(xyz, sph, nullptr, nullptr, n, l_max, pref.data(), buffers.data());
        } else {
            generic_sph<T, true, false, true, 1>(xyz, sph, dsph, nullptr, n, l_max, pref.data(), buffers.data());
        }
    } else {
        if (mode == 0) {
            generic_sph<T, false, false, false, 1>(xyz, sph, nullptr, nullptr, n, l_max, pref.data(), buffers.data());
        } else {
            generic_sph<T, true, false, false, 1>(xyz, sph, dsph, nullptr, n, l_max, pref.data(), buffers.data());
        }
    }
    return 0;
}

} // namespace

extern "C" {

int sphx_ref_compute_f64(const double* xyz, size_t n, int l_max, int normalized, int mode,
                         double* sph, double* dsph, double* ddsph) {
    return run<double>(xyz, n, l_max, normalized, mode, sph, dsph, ddsph);
}

int sphx_ref_compute_f32(const float* xyz, size_t n, int l_max, int normalized, int mode,
                         float* sph, float* dsph, float* ddsph) {
    return run<float>(xyz, n, l_max, normalized, mode, sph, dsph, ddsph);
}

int sphx_ref_recursion_route_f64(const double* xyz, size_t n, int l_max, int normalized, int mode,
                                 double* sph, double* dsph) {
    return run_recursion_route<double>(xyz, n, l_max, normalized, mode, sph, dsph);
}

int sphx_ref_recursion_route_f32(const float* xyz, size_t n, int l_max, int normalized, int mode,
                                 float* sph, float* dsph) {
    return run_recursion_route<float>(xyz, n, l_max, normalized, mode, sph, dsph);
}

void sphx_ref_prefactors_f64(int l_max, double* out) { compute_sph_prefactors<double>(l_max, out); }

void sphx_ref_prefactors_f32(int l_max, float* out) { compute_sph_prefactors<float>(l_max, out); }

int sphx_ref_max_threads(void) { return omp_get_max_threads(); }

} // extern "C"
