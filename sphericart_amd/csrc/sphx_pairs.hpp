// Launch of pairs_kernel, compiled in a translation unit of its own (sphx_pairs.hip).
#ifndef SPHX_PAIRS_HPP
#define SPHX_PAIRS_HPP

#include <hip/hip_runtime.h>

#include "sphx_pairs_plan.hpp"

namespace sphx {

// Enqueue the launch `plan` describes on `stream`, on the current device. `table_F` / `table_Q` are the
// device's prefactor tables (triangular, entry (l, m) at l (l + 1) / 2 + m) in the type of the arithmetic.
// `mode`: 0 values alone, 1 with gradients, 2 with second derivatives too (what the plan was made for).
hipError_t launch_pairs(const PairsLaunch& plan, int mode, bool normalized, const float* table_F,
                        const float* table_Q, const float* xyz, float* sph, float* dsph, float* ddsph,
                        hipStream_t stream);
hipError_t launch_pairs(const PairsLaunch& plan, int mode, bool normalized, const double* table_F,
                        const double* table_Q, const double* xyz, double* sph, double* dsph, double* ddsph,
                        hipStream_t stream);

} // namespace sphx

#endif
