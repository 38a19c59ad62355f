/** Device C++ API of the MI355X (gfx950, HIP) evaluator.
 *
 * Source-compatible with the reference's device classes: same namespace, class
 * names, constructors and member functions as
 * sphericart/include/sphericart_cuda.hpp:33-187 (implementation
 * sphericart/src/sphericart_cuda.cpp:40-196), so callers written against
 * `sphericart::cuda::SphericalHarmonics<T>` / `SolidHarmonics<T>` rebuild
 * against this header unchanged. Every pointer is a device pointer allocated by
 * the caller; `cuda_stream` carries the native stream handle by value (here a
 * `hipStream_t`), `nullptr` meaning the default stream. Calls enqueue work and
 * return without synchronising.
 *
 * This header pulls in no HIP header: the classes sit on the plain C launch
 * layer of sphx_launch.h.
 */
#ifndef SPHERICART_CUDA_HPP
#define SPHERICART_CUDA_HPP

#include <cstddef>

#ifndef SPHERICART_EXPORT
#define SPHERICART_EXPORT __attribute__((visibility("default")))
#endif

namespace sphericart {
namespace cuda {

/**
 * Real spherical harmonics Y_l^m of the direction (x, y, z)/r, for all
 * l <= l_max, stored per point in the order (l, m) = (0,0), (1,-1), (1,0),
 * (1,1), (2,-2), ...
 *
 * Reference: sphericart/include/sphericart_cuda.hpp:33-170.
 */
template <typename T> class SPHERICART_EXPORT SphericalHarmonics {
  public:
    /** @param l_max largest degree to evaluate.
     *  Throws std::runtime_error when no HIP device is usable or l_max
     *  exceeds what the device tables cover. */
    SphericalHarmonics(size_t l_max);
    ~SphericalHarmonics();

    /** sph[n_samples][(l_max+1)^2] from xyz[n_samples][3].
     *  Reference: sphericart/include/sphericart_cuda.hpp:74. */
    void compute(const T* xyz, const size_t n_samples, T* sph, void* cuda_stream = nullptr);

    /** Also dsph[n_samples][3][(l_max+1)^2], the derivatives along x, y, z.
     *  Reference: sphericart/include/sphericart_cuda.hpp:102-104. */
    void compute_with_gradients(
        const T* xyz, const size_t n_samples, T* sph, T* dsph, void* cuda_stream = nullptr
    );

    /** Also ddsph[n_samples][3][3][(l_max+1)^2], the second derivatives.
     *  Reference: sphericart/include/sphericart_cuda.hpp:140-142. */
    void compute_with_hessians(
        const T* xyz, const size_t n_samples, T* sph, T* dsph, T* ddsph, void* cuda_stream = nullptr
    );

    template <typename U> friend class SolidHarmonics;

  private:
    size_t l_max;
    bool normalized;

    void compute_internal(
        const T* xyz,
        const size_t n_samples,
        bool compute_with_gradients,
        bool compute_with_hessian,
        T* sph,
        T* dsph,
        T* ddsph,
        void* cuda_stream
    );
};

/**
 * Solid harmonics r^l Y_l^m: the same polynomials evaluated at (x, y, z)
 * itself. Reference: sphericart/include/sphericart_cuda.hpp:179-187.
 */
template <typename T> class SPHERICART_EXPORT SolidHarmonics : public SphericalHarmonics<T> {
  public:
    SolidHarmonics(size_t l_max);
};

} // namespace cuda
} // namespace sphericart

#endif
