// pairs_kernel (sphx_pairs_kernel.hpp) and its launch: values and derivatives at large l_max, where the rows
// of few points fill LDS. A translation unit of its own, so that it compiles next to the other kernels.

#include <hip/hip_runtime.h>

#include <atomic>

#include "sphx_pairs.hpp"
#include "sphx_pairs_kernel.hpp"

namespace sphx {

namespace {

constexpr int kMaxDevices = 64;

// the kernel may use all of a CU's LDS: said once per kernel and device
template <typename T, int MODE, bool NORM, unsigned NT>
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
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(pairs_kernel<T, MODE, NORM, NT, T>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, limit);
    if (e != hipSuccess) return e;
    allowed[device].store(static_cast<unsigned>(limit), std::memory_order_release);
    return hipSuccess;
}

template <typename T, int MODE, bool NORM>
hipError_t launch(const PairsLaunch& plan, const T* table_F, const T* table_Q, const T* xyz, T* sph, T* dsph,
                  T* ddsph, hipStream_t stream) {
    // (second derivatives in float64 need up to 201 registers per lane: eight waves; in float32 125: sixteen)
    constexpr unsigned NT = MODE == 2 && sizeof(T) == 8 ? 512u : kPairsThreads;
    if (plan.threads > NT || plan.threads % 64u != 0 || plan.workgroups % 8u != 0) {
        return hipErrorInvalidValue; // never planned
    }
    hipError_t e = allow_lds<T, MODE, NORM, NT>(plan.lds_bytes);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((pairs_kernel<T, MODE, NORM, NT, T>), dim3(plan.workgroups), dim3(plan.threads),
                       plan.lds_bytes, stream, plan.g, table_F, table_Q, xyz, sph, dsph, ddsph);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_any(const PairsLaunch& plan, int mode, bool normalized, const T* table_F, const T* table_Q,
                      const T* xyz, T* sph, T* dsph, T* ddsph, hipStream_t stream) {
    if (mode == 0) {
        return normalized ? launch<T, 0, true>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream)
                          : launch<T, 0, false>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream);
    }
    if (mode == 1) {
        return normalized ? launch<T, 1, true>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream)
                          : launch<T, 1, false>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream);
    }
    if (mode == 2) {
        return normalized ? launch<T, 2, true>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream)
                          : launch<T, 2, false>(plan, table_F, table_Q, xyz, sph, dsph, ddsph, stream);
    }
    return hipErrorInvalidValue;
}

} // namespace

hipError_t launch_pairs(const PairsLaunch& plan, int mode, bool normalized, const float* table_F,
                        const float* table_Q, const float* xyz, float* sph, float* dsph, float* ddsph,
                        hipStream_t stream) {
    return launch_any<float>(plan, mode, normalized, table_F, table_Q, xyz, sph, dsph, ddsph, stream);
}

hipError_t launch_pairs(const PairsLaunch& plan, int mode, bool normalized, const double* table_F,
                        const double* table_Q, const double* xyz, double* sph, double* dsph, double* ddsph,
                        hipStream_t stream) {
    return launch_any<double>(plan, mode, normalized, table_F, table_Q, xyz, sph, dsph, ddsph, stream);
}

} // namespace sphx
