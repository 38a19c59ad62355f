// Contractions of the derivative arrays with upstream gradients (gfx950): the
// vector-Jacobian products a reverse-mode caller needs after the forward pass.
//
//   first order   xyz_grad[i][a]  = sum_k dsph[i][a][k] * sph_grad[i][k]
//                 (the reference's backward_kernel, sphericart/src/sphericart_impl.cu:650-684,
//                 launched by spherical_harmonics_backward_cuda_base,
//                 sphericart/src/cuda_base.cpp:156-183)
//   second order  xyz_grad[i][b]  = sum_a sum_k ddsph[i][a][b][k] * dsph_grad[i][a][k]
//                 (what the reference's torch binding writes as
//                 torch.sum(grad.unsqueeze(2) * ddsph, dim=(1, 3)),
//                 sphericart-torch/python/sphericart/torch/register.py:108)
//
// Both read every element of the derivative array once and write three numbers
// per point: they are bound by HBM reads. A group of G lanes (G a power of two
// chosen so that every lane has an element or two of each row) walks over the rows of one
// point, consecutive lanes at consecutive addresses; the groups of a wave take
// consecutive points, so a wave reads one contiguous stretch. Each lane keeps
// three partial sums (one per output component), which a butterfly over the
// group's lanes adds up. The order of the additions is fixed by the geometry,
// so results are reproducible from run to run.

#include <hip/hip_runtime.h>

#include <cstddef>
#include <string>

#include "../../include/sphx_launch.h"

namespace sphx {

extern thread_local std::string t_error;

constexpr unsigned kBackwardThreads = 256;

// SECOND == false: rows = 3, the weight of element (a, k) is w[i][k], it goes to output a.
// SECOND == true:  rows = 9, the weight of element (a, b, k) is w[i][a][k], it goes to output b.
template <typename T, bool SECOND>
__global__ __launch_bounds__(kBackwardThreads) void contraction_kernel(
    const T* __restrict__ d, const T* __restrict__ w, unsigned long long n_samples, unsigned n_total,
    unsigned group, unsigned group_shift, int accumulate, T* __restrict__ out) {
    constexpr unsigned ROWS = SECOND ? 9u : 3u;
    const unsigned points_per_block = kBackwardThreads >> group_shift;
    const unsigned in_group = threadIdx.x & (group - 1u);
    const unsigned long long point =
        static_cast<unsigned long long>(blockIdx.x) * points_per_block + (threadIdx.x >> group_shift);

    T sum0 = 0, sum1 = 0, sum2 = 0;
    if (point < n_samples) {
        // One weight serves three rows (the three output components): three independent sums
        // per lane, and nothing in one trip of the loop waits for the trip before.
        const T* rows = d + point * ROWS * n_total;
        const T* weights = w + point * (SECOND ? 3u : 1u) * n_total;
        for (unsigned a = 0; a < (SECOND ? 3u : 1u); ++a) {
            const T* weight = weights + a * n_total;
            const T* row0 = rows + (3u * a) * n_total;
            const T* row1 = row0 + n_total;
            const T* row2 = row1 + n_total;
#pragma unroll 4
            for (unsigned k = in_group; k < n_total; k += group) {
                const T wk = weight[k];
                sum0 += row0[k] * wk;
                sum1 += row1[k] * wk;
                sum2 += row2[k] * wk;
            }
        }
    }
    // every lane of the wave takes part in the exchange, also those past the last point
    for (unsigned offset = group >> 1; offset > 0; offset >>= 1) {
        sum0 += __shfl_xor(sum0, static_cast<int>(offset));
        sum1 += __shfl_xor(sum1, static_cast<int>(offset));
        sum2 += __shfl_xor(sum2, static_cast<int>(offset));
    }
    if (point < n_samples && in_group < 3u) {
        T value = in_group == 0 ? sum0 : (in_group == 1 ? sum1 : sum2);
        T* target = out + point * 3u + in_group;
        if (accumulate) value += *target;
        *target = value;
    }
}

static int backward_fail(int code, const std::string& what) {
    t_error = what;
    return code;
}

template <typename T, bool SECOND>
static int contract(const T* d, const T* w, size_t n_samples, int n_total, T* out, int accumulate,
                    void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
    if (n_total <= 0) return backward_fail(SPHX_ERR_ARGUMENT, "the row length must be positive");
    if (d == nullptr || w == nullptr || out == nullptr) {
        return backward_fail(SPHX_ERR_ARGUMENT, "null pointer passed to a backward contraction");
    }
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, d);
    if (e != hipSuccess) {
        return backward_fail(SPHX_ERR_HIP, std::string("hipPointerGetAttributes: ") + hipGetErrorString(e));
    }
    int current = 0;
    e = hipGetDevice(&current);
    if (e != hipSuccess) {
        return backward_fail(SPHX_ERR_HIP, std::string("hipGetDevice: ") + hipGetErrorString(e));
    }
    if (attr.device != current) {
        e = hipSetDevice(attr.device);
        if (e != hipSuccess) {
            return backward_fail(SPHX_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
        }
    }
    // lanes per point: a power of two between 4 and 64, one or two elements of a row per lane
    // (l_max = 6, float32, 1M points: 167 us with 32 lanes, 186 us with 16, 238 us with 64)
    unsigned shift = 2;
    while (shift < 6 && (2u << shift) <= static_cast<unsigned>(n_total)) ++shift;
    const unsigned group = 1u << shift;
    const unsigned points_per_block = kBackwardThreads >> shift;
    const unsigned long long blocks = (n_samples + points_per_block - 1) / points_per_block;
    int status = SPHX_OK;
    if (blocks > 0x7fffffffull) {
        status = backward_fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    } else {
        hipLaunchKernelGGL((contraction_kernel<T, SECOND>), dim3(static_cast<unsigned>(blocks)),
                           dim3(kBackwardThreads), 0, reinterpret_cast<hipStream_t>(stream), d, w,
                           static_cast<unsigned long long>(n_samples), static_cast<unsigned>(n_total),
                           group, shift, accumulate, out);
        e = hipGetLastError();
        if (e != hipSuccess) {
            status = backward_fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
        }
    }
    if (attr.device != current) {
        e = hipSetDevice(current);
        if (e != hipSuccess && status == SPHX_OK) {
            status = backward_fail(SPHX_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
        }
    }
    return status;
}

} // namespace sphx

extern "C" {

int sphx_backward_f32(const float* dsph, const float* sph_grad, size_t n_samples, int n_total,
                      float* xyz_grad, int accumulate, void* stream) {
    return sphx::contract<float, false>(dsph, sph_grad, n_samples, n_total, xyz_grad, accumulate, stream);
}

int sphx_backward_f64(const double* dsph, const double* sph_grad, size_t n_samples, int n_total,
                      double* xyz_grad, int accumulate, void* stream) {
    return sphx::contract<double, false>(dsph, sph_grad, n_samples, n_total, xyz_grad, accumulate, stream);
}

int sphx_backward_second_f32(const float* ddsph, const float* dsph_grad, size_t n_samples, int n_total,
                             float* xyz_grad, int accumulate, void* stream) {
    return sphx::contract<float, true>(ddsph, dsph_grad, n_samples, n_total, xyz_grad, accumulate, stream);
}

int sphx_backward_second_f64(const double* ddsph, const double* dsph_grad, size_t n_samples, int n_total,
                             double* xyz_grad, int accumulate, void* stream) {
    return sphx::contract<double, true>(ddsph, dsph_grad, n_samples, n_total, xyz_grad, accumulate, stream);
}

} // extern "C"
