// What every kernel of the launch layer shares: the prefactor tables in constant memory, the
// description of a launch's tiling that the host fills in, and the dynamic LDS array.
#ifndef SPHX_TILING_HPP
#define SPHX_TILING_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "../../include/sphx_launch.h"
#include "sphx_device.hpp"
#include "sphx_geometry.hpp"
#include "sphx_tables.hpp"

namespace sphx {

constexpr int kTableEntries = (SPHX_TABLE_LMAX + 1) * (SPHX_TABLE_LMAX + 2) / 2;

// Every translation unit with kernels has its own copy of the tables (internal linkage: device code is not
// linked across translation units) and fills it through upload_tables below.
static __constant__ float kF32[kTableEntries];
static __constant__ float kQ32[kTableEntries];
static __constant__ double kF64[kTableEntries];
static __constant__ double kQ64[kTableEntries];

template <typename T> __device__ __forceinline__ const T* table_F();
template <typename T> __device__ __forceinline__ const T* table_Q();
template <> __device__ __forceinline__ const float* table_F<float>() { return kF32; }
template <> __device__ __forceinline__ const float* table_Q<float>() { return kQ32; }
template <> __device__ __forceinline__ const double* table_F<double>() { return kF64; }
template <> __device__ __forceinline__ const double* table_Q<double>() { return kQ64; }

// Fill this translation unit's tables of type T on the current device; *F and *Q receive their device addresses.
template <typename T> inline hipError_t upload_tables(const HostTables& t, const T** F, const T** Q) {
    const size_t n = kTableEntries;
    hipError_t e;
    void *f = nullptr, *q = nullptr;
    if constexpr (sizeof(T) == 4) {
        e = hipMemcpyToSymbol(HIP_SYMBOL(kF32), t.f32.data(), n * sizeof(float));
        if (e == hipSuccess) e = hipMemcpyToSymbol(HIP_SYMBOL(kQ32), t.f32.data() + n, n * sizeof(float));
        if (e == hipSuccess) e = hipGetSymbolAddress(&f, HIP_SYMBOL(kF32));
        if (e == hipSuccess) e = hipGetSymbolAddress(&q, HIP_SYMBOL(kQ32));
    } else {
        e = hipMemcpyToSymbol(HIP_SYMBOL(kF64), t.f64.data(), n * sizeof(double));
        if (e == hipSuccess) e = hipMemcpyToSymbol(HIP_SYMBOL(kQ64), t.f64.data() + n, n * sizeof(double));
        if (e == hipSuccess) e = hipGetSymbolAddress(&f, HIP_SYMBOL(kF64));
        if (e == hipSuccess) e = hipGetSymbolAddress(&q, HIP_SYMBOL(kQ64));
    }
    if (F != nullptr) *F = static_cast<const T*>(f);
    if (Q != nullptr) *Q = static_cast<const T*>(q);
    return e;
}

extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

// Output lines are written once and never read back by the kernel: store them with the
// non-temporal hint (measured 10-20 % faster than plain stores here).
#ifndef SPHX_STREAMING_STORES
#define SPHX_STREAMING_STORES true
#endif

// LDS loads a flushing wave of the recursion kernel keeps in flight
#ifndef SPHX_FLUSH_UNROLL
#define SPHX_FLUSH_UNROLL 4
#endif

} // namespace sphx

#endif
