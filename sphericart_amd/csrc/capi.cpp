// The twenty sphericart_cuda_* C entry points over the device classes.
//
// Error convention of the reference (sphericart/src/sphericart-capi.cpp:637-700):
// `new` maps any exception to a null handle, `delete` swallows exceptions,
// `compute*` prints "fatal error: <what>" on stdout and aborts.

#include "../../include/sphericart.h"

#include <cstdio>
#include <cstdlib>
#include <exception>

namespace {

template <typename Calculator> Calculator* make(size_t l_max) {
    try {
        return new Calculator(l_max);
    } catch (...) {
        return nullptr;
    }
}

template <typename Calculator> void destroy(Calculator* calculator) {
    try {
        delete calculator;
    } catch (...) {
    }
}

template <typename Body> void guarded(Body&& body) {
    try {
        body();
    } catch (const std::exception& e) {
        std::printf("fatal error: %s\n", e.what());
        std::fflush(stdout);
        std::abort();
    } catch (...) {
        std::printf("fatal error: unknown exception type\n");
        std::fflush(stdout);
        std::abort();
    }
}

} // namespace

#define SPHX_DEFINE_FAMILY(NAME, SUFFIX, CALC, T)                                                  \
    extern "C" CALC* sphericart_cuda_##NAME##_new##SUFFIX(size_t l_max) {                          \
        return make<CALC>(l_max);                                                                  \
    }                                                                                              \
    extern "C" void sphericart_cuda_##NAME##_delete##SUFFIX(CALC* calculator) {                    \
        destroy(calculator);                                                                       \
    }                                                                                              \
    extern "C" void sphericart_cuda_##NAME##_compute_array##SUFFIX(                                \
        CALC* calculator, const T* xyz, size_t n_samples, T* sph, void* cuda_stream                \
    ) {                                                                                            \
        guarded([&] { calculator->compute(xyz, n_samples, sph, cuda_stream); });                   \
    }                                                                                              \
    extern "C" void sphericart_cuda_##NAME##_compute_array_with_gradients##SUFFIX(                 \
        CALC* calculator, const T* xyz, size_t n_samples, T* sph, T* dsph, void* cuda_stream       \
    ) {                                                                                            \
        guarded([&] {                                                                              \
            calculator->compute_with_gradients(xyz, n_samples, sph, dsph, cuda_stream);            \
        });                                                                                        \
    }                                                                                              \
    extern "C" void sphericart_cuda_##NAME##_compute_array_with_hessians##SUFFIX(                  \
        CALC* calculator, const T* xyz, size_t n_samples, T* sph, T* dsph, T* ddsph,               \
        void* cuda_stream                                                                          \
    ) {                                                                                            \
        guarded([&] {                                                                              \
            calculator->compute_with_hessians(xyz, n_samples, sph, dsph, ddsph, cuda_stream);      \
        });                                                                                        \
    }

SPHX_DEFINE_FAMILY(spherical_harmonics, , sphericart_cuda_spherical_harmonics_calculator_t, double)
SPHX_DEFINE_FAMILY(spherical_harmonics, _f, sphericart_cuda_spherical_harmonics_calculator_f_t, float)
SPHX_DEFINE_FAMILY(solid_harmonics, , sphericart_cuda_solid_harmonics_calculator_t, double)
SPHX_DEFINE_FAMILY(solid_harmonics, _f, sphericart_cuda_solid_harmonics_calculator_f_t, float)
