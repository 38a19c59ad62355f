// pairs_kernel (sphx_pairs_kernel.hpp) and its launch: values and gradients at large l_max, where the rows
// of few points fill LDS. A translation unit of its own, so that it compiles next to the other kernels.

#include <hip/hip_runtime.h>

#include <atomic>

#include "sphx_pairs.hpp"
#include "sphx_pairs_kernel.hpp"

namespace sphx {

namespace {

constexpr int kMaxDevices = 64;

// the kernel may use all of a CU's LDS: said once per kernel and device
template <typename T, bool NORM>
hipError_t allow_lds(unsigned lds_bytes) {
    static std::atomic<unsigned> allowed[kMaxDevices];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (allowed[device].load(std::memory_order_acquire) >= lds_bytes) return hipSuccess;
    int limit = 0;
    e = hipDeviceGetAttribute(&limit, hipDeviceAttributeMaxSharedMemoryPerBlock, device);
    if (e != hipSuccess) return e;
    if (static_cast<unsigned>(limit) < lds_bytes) return hipErrorInvalidValue;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(pairs_kernel<T, NORM, T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, limit);
    if (e != hipSuccess) return e;
    allowed[device].store(static_cast<unsigned>(limit), std::memory_order_release);
    return hipSuccess;
}

template <typename T, bool NORM>
hipError_t launch(const PairsLaunch& plan, const T* table_F, const T* table_Q, const T* xyz, T* sph, T* dsph,
                  hipStream_t stream) {
    if (plan.threads > kPairsThreads || plan.threads % 64u != 0 || plan.workgroups % 8u != 0) {
        return hipErrorInvalidValue; // never planned
    }
    hipError_t e = allow_lds<T, NORM>(plan.lds_bytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((pairs_kernel<T, NORM, T>), dim3(plan.workgroups), dim3(plan.threads), plan.lds_bytes, stream,
                       plan.g, table_F, table_Q, xyz, sph, dsph);
    return hipGetLastError();
}

} // namespace

hipError_t launch_pairs(const PairsLaunch& plan, bool normalized, const float* table_F, const float* table_Q,
                        const float* xyz, float* sph, float* dsph, hipStream_t stream) {
    return normalized ? launch<float, true>(plan, table_F, table_Q, xyz, sph, dsph, stream)
                      : launch<float, false>(plan, table_F, table_Q, xyz, sph, dsph, stream);
}

hipError_t launch_pairs(const PairsLaunch& plan, bool normalized, const double* table_F, const double* table_Q,
                        const double* xyz, double* sph, double* dsph, hipStream_t stream) {
    return normalized ? launch<double, true>(plan, table_F, table_Q, xyz, sph, dsph, stream)
                      : launch<double, false>(plan, table_F, table_Q, xyz, sph, dsph, stream);
}

} // namespace sphx
