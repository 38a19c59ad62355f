// The launches of the forward kernels, as templates over the arithmetic type and the derivatives asked for. A
// translation unit includes this and instantiates dispatch_forward<T, MODE> (or dispatch_wide<MODE>) for the one
// combination it is there for, together with the uploader of its constant tables.
#ifndef SPHX_DISPATCH_HPP
#define SPHX_DISPATCH_HPP

#include <hip/hip_runtime.h>

#include "sphx_runtime.hpp"

#include "sphx_device.hpp"
#include "sphx_tiling.hpp"
#include "sphx_closed_form_kernel.hpp"
#include "sphx_lane_kernels.hpp"
#include "sphx_recursion_kernel.hpp"
#include "sphx_pairs.hpp"

namespace sphx {

template <typename T, int MODE, bool NORM, int H, bool PREFIX>
static hipError_t launch_closed(const Launch& l, const T* xyz, T* sph, T* dsph, T* ddsph,
                                hipStream_t stream) {
    auto kernel = closed_form_kernel<T, MODE, NORM, H, PREFIX>;
    if (l.lds_bytes > 64u * 1024u) {
        unsigned unused = 0;
        hipError_t e = kernel_facts(reinterpret_cast<const void*>(kernel), l.threads, l.lds_bytes, &unused);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3(l.workgroups), dim3(l.threads), l.lds_bytes, stream, l.g, xyz,
                       sph, dsph, ddsph);
    return hipGetLastError();
}

template <typename X> struct AsGiven {
    using type = X; // a parameter of this type takes no part in template argument deduction
};

// Workgroups of 1024 threads (one per CU, all of its LDS) exist for all but the fused product and those
// second derivatives in float64 whose entry jobs need more registers than sixteen waves leave a lane (128): the
// two sides of an (l, m) pair as one job (163-231), and for normalised harmonics the sides as two jobs taken
// point by point (173; as one list ordered by kind 129, which the compiler brings down to 128).
template <typename T, int MODE, bool VJP, bool NORM = true, bool SPLIT = false, bool LIST = false>
constexpr bool kLargeGroups =
    !VJP && (MODE <= 1 || (MODE == 2 && sizeof(T) == 4) || (MODE == 2 && SPLIT && (!NORM || LIST)));

template <typename T, int MODE, bool NORM, bool WHOLE, bool SPLIT, bool VJP = false, bool LIST = false,
          typename O = T, unsigned NT = kRecursionThreads, bool TOGETHER = false>
static hipError_t launch_recursion(const Launch& l, const typename AsGiven<O>::type* xyz,
                                   typename AsGiven<O>::type* sph, typename AsGiven<O>::type* dsph,
                                   typename AsGiven<O>::type* ddsph, hipStream_t stream) {
    if constexpr (!VJP && !LIST) {
        // the variant whose entry lanes take the jobs of a tile as one list
        if (l.g.points_per_pass == 0) {
            return launch_recursion<T, MODE, NORM, WHOLE, SPLIT, false, true, O, NT, TOGETHER>(l, xyz, sph, dsph, ddsph, stream);
        }
    }
    if constexpr (NT == kRecursionThreads && kLargeGroups<T, MODE, VJP, NORM, SPLIT, LIST>) {
        if (l.threads == 2 * kRecursionThreads) {
            return launch_recursion<T, MODE, NORM, WHOLE, SPLIT, VJP, LIST, O, 2 * kRecursionThreads, TOGETHER>(
                l, xyz, sph, dsph, ddsph, stream);
        }
    }
    if constexpr (sizeof(T) == 8 && !TOGETHER) {
        // the variant whose recursions run next to the entries
        if (l.g.together != 0) {
            return launch_recursion<T, MODE, NORM, WHOLE, SPLIT, VJP, LIST, O, NT, true>(l, xyz, sph, dsph, ddsph, stream);
        }
    }
    if ((l.g.together != 0) != TOGETHER) return hipErrorInvalidValue; // never planned
    if (l.threads != NT) return hipErrorInvalidValue; // never planned
    auto kernel = recursion_kernel<T, MODE, NORM, WHOLE, SPLIT, VJP, LIST, O, NT, TOGETHER>;
    // The workgroups are persistent: launch exactly as many as are resident at once (registers
    // may allow fewer per CU than LDS does), or the last ones would run alone after the rest.
    unsigned workgroups = l.workgroups;
    unsigned cap = 0;
    hipError_t e = kernel_facts(reinterpret_cast<const void*>(kernel), l.threads, l.lds_bytes, &cap);
    if (e != hipSuccess) return e;
    if (cap >= 8 && cap < workgroups) workgroups = cap;
    hipLaunchKernelGGL(kernel, dim3(workgroups), dim3(l.threads), l.lds_bytes, stream, l.g, xyz,
                       sph, dsph, ddsph);
    return hipGetLastError();
}

template <typename T, int MODE, bool NORM>
static hipError_t dispatch(const Plan& plan, const DeviceState& device, const T* xyz, T* sph, T* dsph, T* ddsph,
                           hipStream_t stream) {
    if (plan.pairs) {
        {
            const T *F, *Q;
            if constexpr (sizeof(T) == 4) {
                F = device.F32;
                Q = device.Q32;
            } else {
                F = device.F64;
                Q = device.Q64;
            }
            return launch_pairs(plan.pairs_launch, MODE, NORM, F, Q, xyz, sph, dsph, ddsph, stream);
        }
    }
    if (plan.lanes) {
        if constexpr (MODE == 0) {
            const Launch& l = plan.closed;
            auto kernel = l.g.points_per_pass == 4   ? values_kernel<T, NORM, 4>
                          : l.g.points_per_pass == 2 ? (l.threads > 512 ? values_kernel<T, NORM, 2, 1024> : values_kernel<T, NORM, 2>)
                          : l.threads > 512          ? values_kernel<T, NORM, 1, 1024>
                                                     : values_kernel<T, NORM, 1>;
            if (l.threads > (l.g.points_per_pass == 4 ? 512u : 1024u)) return hipErrorInvalidValue; // never planned
            if (l.lds_bytes > 64u * 1024u) {
                unsigned unused = 0;
                hipError_t e = kernel_facts(reinterpret_cast<const void*>(kernel), l.threads, l.lds_bytes, &unused);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(kernel, dim3(l.workgroups), dim3(l.threads), l.lds_bytes, stream, l.g, xyz, sph);
            return hipGetLastError();
        }
        if constexpr (MODE == 1) {
            const Launch& l = plan.closed;
            if (l.g.l_max < 4) return hipErrorInvalidValue; // never planned
            if (l.threads > (l.g.l_max >= 6 ? 1024u : 512u)) return hipErrorInvalidValue; // never planned
            auto kernel = l.g.l_max >= 6   ? (l.threads > 512 ? gradients_lanes_kernel<T, NORM, 6, 1024>
                                                              : gradients_lanes_kernel<T, NORM, 6>)
                          : l.g.l_max == 5 ? gradients_lanes_kernel<T, NORM, 5>
                                           : gradients_lanes_kernel<T, NORM, 4>;
            if (l.lds_bytes > 64u * 1024u) {
                unsigned unused = 0;
                hipError_t e = kernel_facts(reinterpret_cast<const void*>(kernel), l.threads, l.lds_bytes, &unused);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(kernel, dim3(l.workgroups), dim3(l.threads), l.lds_bytes, stream, l.g, xyz, sph,
                               dsph);
            return hipGetLastError();
        }
        if constexpr (MODE == 2) {
            const Launch& l = plan.closed;
            if (l.threads > hessian_lane_threads<T>()) return hipErrorInvalidValue; // never planned
            auto kernel = hessians_lanes_kernel<T, NORM>;
            if (l.lds_bytes > 64u * 1024u) {
                unsigned unused = 0;
                hipError_t e = kernel_facts(reinterpret_cast<const void*>(kernel), l.threads, l.lds_bytes, &unused);
                if (e != hipSuccess) return e;
            }
            hipLaunchKernelGGL(kernel, dim3(l.workgroups), dim3(l.threads), l.lds_bytes, stream, l.g, xyz, sph,
                               dsph, ddsph);
            return hipGetLastError();
        }
        return hipErrorInvalidValue;
    }
    if (!plan.closed_only) {
        if constexpr (MODE == 2) {
            if (plan.split_sides) {
                return launch_recursion<T, MODE, NORM, true, true>(plan.rec, xyz, sph, dsph, ddsph, stream);
            }
            return launch_recursion<T, MODE, NORM, true, false>(plan.rec, xyz, sph, dsph, ddsph, stream);
        } else {
            if (plan.whole) {
                return launch_recursion<T, MODE, NORM, true, false>(plan.rec, xyz, sph, dsph, ddsph, stream);
            }
            if (plan.rec.g.prefix_inside != 0) {
                return launch_recursion<T, MODE, NORM, false, false>(plan.rec, xyz, sph, dsph, ddsph, stream);
            }
            // the two kernels write disjoint parts of every row
            hipError_t e = launch_closed<T, MODE, NORM, 6, true>(plan.closed, xyz, sph, dsph, ddsph, stream);
            if (e != hipSuccess) return e;
            return launch_recursion<T, MODE, NORM, false, false>(plan.rec, xyz, sph, dsph, ddsph, stream);
        }
    }
    const Launch& l = plan.closed;
    switch (l.g.l_max) {
    case 0:
        return launch_closed<T, MODE, NORM, 0, false>(l, xyz, sph, dsph, ddsph, stream);
    case 1:
        return launch_closed<T, MODE, NORM, 1, false>(l, xyz, sph, dsph, ddsph, stream);
    default:
        break;
    }
    if constexpr (MODE < 2) {
        switch (l.g.l_max) {
        case 2:
            return launch_closed<T, MODE, NORM, 2, false>(l, xyz, sph, dsph, ddsph, stream);
        case 3:
            return launch_closed<T, MODE, NORM, 3, false>(l, xyz, sph, dsph, ddsph, stream);
        case 4:
            return launch_closed<T, MODE, NORM, 4, false>(l, xyz, sph, dsph, ddsph, stream);
        case 5:
            return launch_closed<T, MODE, NORM, 5, false>(l, xyz, sph, dsph, ddsph, stream);
        case 6:
            return launch_closed<T, MODE, NORM, 6, false>(l, xyz, sph, dsph, ddsph, stream);
        default:
            break;
        }
    }
    return hipErrorInvalidValue;
}

template <int MODE, bool NORM>
static hipError_t dispatch_wide_as(const Plan& plan, const float* xyz, float* sph, float* dsph, float* ddsph,
                                hipStream_t stream) {
    if constexpr (MODE == 2) {
        if (plan.split_sides) {
            return launch_recursion<double, 2, NORM, true, true, false, false, float>(plan.rec, xyz, sph, dsph, ddsph, stream);
        }
        return launch_recursion<double, 2, NORM, true, false, false, false, float>(plan.rec, xyz, sph, dsph, ddsph, stream);
    } else {
        if (plan.whole) {
            return launch_recursion<double, MODE, NORM, true, false, false, false, float>(plan.rec, xyz, sph, dsph, ddsph, stream);
        }
        return launch_recursion<double, MODE, NORM, false, false, false, false, float>(plan.rec, xyz, sph, dsph, ddsph, stream);
    }
}


template <typename T, int MODE>
hipError_t dispatch_forward(const Plan& plan, const DeviceState& device, bool normalized, const T* xyz, T* sph,
                            T* dsph, T* ddsph, hipStream_t stream) {
    return normalized ? dispatch<T, MODE, true>(plan, device, xyz, sph, dsph, ddsph, stream)
                      : dispatch<T, MODE, false>(plan, device, xyz, sph, dsph, ddsph, stream);
}

template <typename T, int MODE> hipError_t upload_forward_tables(const HostTables& t, const T** F, const T** Q) {
    return upload_tables<T>(t, F, Q);
}

template <int MODE>
hipError_t dispatch_wide(const Plan& plan, bool normalized, const float* xyz, float* sph, float* dsph, float* ddsph,
                         hipStream_t stream) {
    return normalized ? dispatch_wide_as<MODE, true>(plan, xyz, sph, dsph, ddsph, stream)
                      : dispatch_wide_as<MODE, false>(plan, xyz, sph, dsph, ddsph, stream);
}

template <int MODE> hipError_t upload_wide_tables(const HostTables& t) {
    return upload_tables<double>(t, nullptr, nullptr);
}

} // namespace sphx

#endif
