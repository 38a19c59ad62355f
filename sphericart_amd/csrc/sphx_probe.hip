// Yardsticks for the benchmark (include/sphx_launch.h, sphx_probe_*): what a launch of nothing costs, how fast
// plain stores fill HBM, and what a call of the evaluator costs the host. None of it is on the path of an
// evaluation.

#include <hip/hip_runtime.h>

#include <chrono>
#include <string>

#include "../../include/sphericart.h"
#include "../../include/sphx_launch.h"
#include "sphx_plan.hpp"

namespace sphx {

__global__ void nothing_kernel() {}

// One 16-byte store per lane, consecutive lanes at consecutive addresses, a workgroup per 4 KB: of the plain
// fills measured on an MI355X (persistent workgroups that stride through the buffer or through an eighth of it,
// chunks per workgroup, streaming or ordinary stores, hipMemsetAsync) this one is the fastest, 6.9 TB/s on 1 GB.
typedef unsigned int Words4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void fill_kernel(Words4* __restrict__ out, unsigned long long vectors) {
    const unsigned long long i = static_cast<unsigned long long>(blockIdx.x) * 256ull + threadIdx.x;
    const Words4 value = {0x3f800000u, 0x3f800000u, 0x3f800000u, 0x3f800000u};
    if (i < vectors) out[i] = value;
}

} // namespace sphx

extern "C" {

int sphx_probe_empty_launch(void* stream) {
    hipLaunchKernelGGL(sphx::nothing_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream));
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPHX_OK : sphx::fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
}

int sphx_probe_fill(void* out, size_t bytes, void* stream) {
    if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15u) != 0 || bytes % 16 != 0) {
        return sphx::fail(SPHX_ERR_ARGUMENT, "sphx_probe_fill: a buffer aligned to 16 bytes, a multiple of 16 long");
    }
    const unsigned long long vectors = bytes / 16;
    if (vectors == 0) return SPHX_OK;
    const unsigned long long want = (vectors + 255ull) / 256ull;
    if (want > 0x7fffffffull) return sphx::fail(SPHX_ERR_UNSUPPORTED, "sphx_probe_fill: at most 2^31 workgroups of 4 KB");
    const unsigned workgroups = static_cast<unsigned>(want);
    hipLaunchKernelGGL(sphx::fill_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       static_cast<sphx::Words4*>(out), vectors);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? SPHX_OK : sphx::fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
}

int sphx_probe_host_cost_f64(int through, const double* xyz, size_t n_samples, int l_max, double* sph, double* dsph,
                             void* stream, int calls, double* seconds_per_call) {
    if (calls <= 0 || seconds_per_call == nullptr) return sphx::fail(SPHX_ERR_ARGUMENT, "sphx_probe_host_cost_f64: calls > 0");
    sphericart_cuda_spherical_harmonics_calculator_t* calculator = nullptr;
    if (through == 1) {
        calculator = sphericart_cuda_spherical_harmonics_new(static_cast<size_t>(l_max));
        if (calculator == nullptr) return sphx::fail(SPHX_ERR_HIP, "sphx_probe_host_cost_f64: no calculator");
    } else if (through != 0) {
        return sphx::fail(SPHX_ERR_ARGUMENT, "sphx_probe_host_cost_f64: through = 0 (sphx_forward_f64) or 1 (sphericart_cuda_*)");
    }
    int status = SPHX_OK;
    const auto begin = std::chrono::steady_clock::now();
    for (int i = 0; i < calls && status == SPHX_OK; ++i) {
        if (through == 0) {
            status = sphx_forward_f64(xyz, n_samples, l_max, 1, 1, sph, dsph, nullptr, stream);
        } else {
            sphericart_cuda_spherical_harmonics_compute_array_with_gradients(calculator, xyz, n_samples, sph, dsph, stream);
        }
    }
    const auto end = std::chrono::steady_clock::now();
    if (calculator != nullptr) sphericart_cuda_spherical_harmonics_delete(calculator);
    *seconds_per_call = std::chrono::duration<double>(end - begin).count() / calls;
    return status;
}

} // extern "C"
