// sphericart::cuda::SphericalHarmonics<T> / SolidHarmonics<T> on top of the C
// launch layer. Plain host C++: no HIP header is included here.
//
// Behaviour follows the reference device classes
// (sphericart/src/sphericart_cuda.cpp:40-196): zero samples return before any
// pointer is looked at (:85-89), null output pointers raise
// std::runtime_error with the reference's messages (:91-113), the solid class
// is the spherical one with normalisation switched off (:186-189).

#include "../../include/sphericart_cuda.hpp"

#include <stdexcept>
#include <string>

#include "../../include/sphx_launch.h"

using namespace sphericart::cuda;

template <typename T> SphericalHarmonics<T>::SphericalHarmonics(size_t l_max) {
    if (sphx_device_count() <= 0) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics: no usable HIP device (" +
            std::string(sphx_last_error()) + ")"
        );
    }
    if (l_max > SPHX_TABLE_LMAX) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics: l_max = " + std::to_string(l_max) +
            " exceeds the largest degree of the device prefactor tables (" +
            std::to_string(SPHX_TABLE_LMAX) + ")"
        );
    }
    this->l_max = l_max;
    this->normalized = true;
}

template <typename T> SphericalHarmonics<T>::~SphericalHarmonics() {}

namespace {

inline int launch(const float* xyz, size_t n, int l_max, bool normalized, int mode, float* sph,
                  float* dsph, float* ddsph, void* stream) {
    return sphx_forward_f32(xyz, n, l_max, normalized ? 1 : 0, mode, sph, dsph, ddsph, stream);
}

inline int launch(const double* xyz, size_t n, int l_max, bool normalized, int mode, double* sph,
                  double* dsph, double* ddsph, void* stream) {
    return sphx_forward_f64(xyz, n, l_max, normalized ? 1 : 0, mode, sph, dsph, ddsph, stream);
}

} // namespace

template <typename T>
void SphericalHarmonics<T>::compute_internal(
    const T* xyz,
    const size_t n_samples,
    bool compute_with_gradients,
    bool compute_with_hessian,
    T* sph,
    T* dsph,
    T* ddsph,
    void* cuda_stream
) {
    if (n_samples == 0) {
        // empty inputs may legitimately come with null pointers
        return;
    }

    if (sph == nullptr) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics::compute expected "
            "sph ptr initialised, instead nullptr found. Initialise "
            "sph with hipMalloc."
        );
    }

    if (compute_with_gradients && dsph == nullptr) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics::compute expected "
            "dsph != nullptr since compute_with_gradients = true. "
            "initialise dsph with hipMalloc."
        );
    }

    if (compute_with_hessian && ddsph == nullptr) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics::compute expected "
            "ddsph != nullptr since compute_with_hessian = true. "
            "initialise ddsph with hipMalloc."
        );
    }

    const int mode = compute_with_hessian ? SPHX_HESSIANS
                                          : (compute_with_gradients ? SPHX_GRADIENTS : SPHX_VALUES);
    const int status = launch(
        xyz, n_samples, static_cast<int>(this->l_max), this->normalized, mode, sph, dsph, ddsph,
        cuda_stream
    );
    if (status != SPHX_OK) {
        throw std::runtime_error(
            "sphericart::cuda::SphericalHarmonics::compute: " + std::string(sphx_last_error())
        );
    }
}

template <typename T>
void SphericalHarmonics<T>::compute(const T* xyz, const size_t n_samples, T* sph, void* cuda_stream) {
    this->compute_internal(xyz, n_samples, false, false, sph, nullptr, nullptr, cuda_stream);
}

template <typename T>
void SphericalHarmonics<T>::compute_with_gradients(
    const T* xyz, const size_t n_samples, T* sph, T* dsph, void* cuda_stream
) {
    this->compute_internal(xyz, n_samples, true, false, sph, dsph, nullptr, cuda_stream);
}

template <typename T>
void SphericalHarmonics<T>::compute_with_hessians(
    const T* xyz, const size_t n_samples, T* sph, T* dsph, T* ddsph, void* cuda_stream
) {
    this->compute_internal(xyz, n_samples, true, true, sph, dsph, ddsph, cuda_stream);
}

template <typename T>
SolidHarmonics<T>::SolidHarmonics(size_t l_max) : SphericalHarmonics<T>(l_max) {
    this->normalized = false;
}

template class sphericart::cuda::SphericalHarmonics<float>;
template class sphericart::cuda::SphericalHarmonics<double>;
template class sphericart::cuda::SolidHarmonics<float>;
template class sphericart::cuda::SolidHarmonics<double>;
