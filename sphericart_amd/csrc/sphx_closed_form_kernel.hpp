// closed_form_kernel: l <= 6 (l <= 1 with second derivatives) in closed form, one point per lane.
#ifndef SPHX_CLOSED_FORM_KERNEL_HPP
#define SPHX_CLOSED_FORM_KERNEL_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sphx_tiling.hpp"

namespace sphx {

// ---------------------------------------------------------------------------
// l <= H in closed form. One wave per workgroup, one point per lane, 64 points
// per workgroup.
//
// The finished numbers of a point stay in the lane's VGPRs; LDS is only the
// transposition buffer between "one point per lane" and "consecutive addresses
// per lane". The 64 points go through the buffer in PHASES passes of
// 64 / PHASES points each when all of them do not fit.
//
// PREFIX == false: l_max == H. The slice of every output array that a pass
// covers is one contiguous run, streamed out with 16-byte stores.
// PREFIX == true: l_max > H; only the first (H+1)^2 entries of every component
// row are produced here (the recursion kernel fills in the rest), so the runs
// are (H+1)^2 long and ny apart.
// ---------------------------------------------------------------------------
// (The LDS one pass may use, SPHX_PHASE_LDS_BUDGET, and the padding of the rows: sphx_geometry.hpp. 52 KB lets
// three workgroups share a CU.)

template <typename T, int MODE, bool NORM, int H, bool PREFIX>
__global__ __launch_bounds__(64) void closed_form_kernel(Tiling g, const T* __restrict__ xyz,
                                                        T* __restrict__ sph, T* __restrict__ dsph,
                                                        T* __restrict__ ddsph) {
    constexpr unsigned PHASES = closed_form_phases(sizeof(T), MODE, H);
    constexpr unsigned PER = 64 / PHASES;
    constexpr unsigned NY = (H + 1) * (H + 1);
    constexpr unsigned PAD = closed_form_pad(H);
    // LDS: [PER][NY + PAD] values, then [PER][3 NY + PAD] gradients, then [PER][9 NY + PAD]
    constexpr unsigned OFF_D = (PER * (NY + PAD) + 3u) & ~3u;
    constexpr unsigned OFF_DD = (OFF_D + PER * (3 * NY + PAD) + 3u) & ~3u;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    // Workgroups are handed to the 8 XCDs round-robin; give each XCD one contiguous stretch of
    // points, so that what one XCD writes at any moment is a compact window of each array
    // (measured: 6 % faster than the identity mapping).
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned long long first = static_cast<unsigned long long>(group) * 64;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < 64ull ? static_cast<unsigned>(left) : 64u;

    Entry<T> E[NY];
    if (tid < valid) {
        const Point<T> p = load_point<T, NORM>(xyz + (first + tid) * 3);
        closed_form_entries<T, MODE, NORM, H>(p, E);
    }
#pragma unroll
    for (unsigned phase = 0; phase < PHASES; ++phase) {
        const unsigned base = phase * PER;
        if (base >= valid) break; // uniform across the wave
        if (phase > 0) __syncthreads();
        if (tid >= base && tid < base + PER && tid < valid) {
            const unsigned s = tid - base;
            Rows<T> rows;
            rows.ny = NY;
            rows.sph = lds + s * (NY + PAD);
            rows.dsph = lds + OFF_D + s * (3 * NY + PAD);
            rows.ddsph = lds + OFF_DD + s * (9 * NY + PAD);
#pragma unroll
            for (unsigned k = 0; k < NY; ++k) {
                put<T, MODE>(rows, k, E[k]);
            }
        }
        __syncthreads();
        const unsigned count = valid - base < PER ? valid - base : PER;
        const unsigned long long at = first + base;
        if constexpr (!PREFIX) {
            copy_out<T, SPHX_STREAMING_STORES, PAD != 0>(lds, sph + at * NY, count * NY, NY, PAD,
                                                         magic_of(NY), tid, 64);
            if constexpr (MODE >= 1) {
                copy_out<T, SPHX_STREAMING_STORES, PAD != 0>(lds + OFF_D, dsph + at * 3 * NY,
                                                             count * 3 * NY, 3 * NY, PAD,
                                                             magic_of(3 * NY), tid, 64);
            }
            if constexpr (MODE == 2) {
                copy_out<T, SPHX_STREAMING_STORES, PAD != 0>(lds + OFF_DD, ddsph + at * 9 * NY,
                                                             count * 9 * NY, 9 * NY, PAD,
                                                             magic_of(9 * NY), tid, 64);
            }
        } else {
            const unsigned ny = g.ny;
            copy_prefixes<T, SPHX_STREAMING_STORES, NY, 1>(lds, sph + at * ny, count, ny, PAD, tid, 64);
            if constexpr (MODE >= 1) {
                copy_prefixes<T, SPHX_STREAMING_STORES, NY, 3>(lds + OFF_D, dsph + at * 3 * ny, count,
                                                              ny, PAD, tid, 64);
            }
            if constexpr (MODE == 2) {
                copy_prefixes<T, SPHX_STREAMING_STORES, NY, 9>(lds + OFF_DD, ddsph + at * 9 * ny,
                                                              count, ny, PAD, tid, 64);
            }
        }
    }
}

} // namespace sphx

#endif
