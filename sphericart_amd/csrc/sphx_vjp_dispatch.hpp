// The launches of the fused product (sphx_vjp_*), as templates over the arithmetic type; sphx_vjp_f32.hip and
// sphx_vjp_f64.hip instantiate dispatch_vjp<T> and the uploader of their constant tables.
#ifndef SPHX_VJP_DISPATCH_HPP
#define SPHX_VJP_DISPATCH_HPP

#include "sphx_dispatch.hpp"
#include "sphx_vjp_kernels.hpp"

namespace sphx {

// l_max > 6: the gradient kernels with the contraction in place of the flush; the closed forms
// either inside the recursion kernel or, when its tiles are small, in a launch of their own that
// stores the sum over l <= 6, to which the recursion kernel then adds the rest.
template <typename T, bool NORM>
static hipError_t launch_vjp_recursion(const Plan& plan, const T* xyz, const T* sph_grad, T* xyz_grad,
                                       int accumulate, hipStream_t stream);

template <typename T, bool NORM, int H>
static hipError_t launch_vjp(const Launch& l, const T* xyz, const T* sph_grad, T* xyz_grad,
                             int accumulate, hipStream_t stream) {
    constexpr unsigned NY = (H + 1) * (H + 1);
    const unsigned lds_bytes = 64u * (NY + closed_form_pad(H)) * static_cast<unsigned>(sizeof(T));
    hipLaunchKernelGGL((closed_form_vjp_kernel<T, NORM, H>), dim3(l.workgroups), dim3(64), lds_bytes,
                       stream, l.g, xyz, sph_grad, xyz_grad, accumulate);
    return hipGetLastError();
}

template <typename T, bool NORM>
static hipError_t dispatch_vjp_closed(const Launch& l, int l_max, const T* xyz, const T* sph_grad,
                               T* xyz_grad, int accumulate, hipStream_t stream) {
    switch (l_max) {
    case 0: return launch_vjp<T, NORM, 0>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 1: return launch_vjp<T, NORM, 1>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 2: return launch_vjp<T, NORM, 2>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 3: return launch_vjp<T, NORM, 3>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 4: return launch_vjp<T, NORM, 4>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 5: return launch_vjp<T, NORM, 5>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    case 6: return launch_vjp<T, NORM, 6>(l, xyz, sph_grad, xyz_grad, accumulate, stream);
    default: return hipErrorInvalidValue;
    }
}

template <typename T, bool NORM>
static hipError_t launch_vjp_recursion(const Plan& plan, const T* xyz, const T* sph_grad, T* xyz_grad,
                                       int accumulate, hipStream_t stream) {
    Launch rec = plan.rec;
    rec.g.vjp_accumulate = accumulate != 0;
    // the kernel reads its `sph` argument and writes three numbers per point through `dsph`
    T* upstream = const_cast<T*>(sph_grad);
    if (plan.whole) {
        return launch_recursion<T, 1, NORM, true, false, true>(rec, xyz, upstream, xyz_grad, nullptr, stream);
    }
    hipError_t e = launch_vjp<T, NORM, 6>(plan.closed, xyz, sph_grad, xyz_grad, accumulate, stream);
    if (e != hipSuccess) return e;
    return launch_recursion<T, 1, NORM, false, false, true>(rec, xyz, upstream, xyz_grad, nullptr, stream);
}

template <typename T>
hipError_t dispatch_vjp(const VjpPlan& planned, int l_max, bool normalized, const T* xyz, const T* sph_grad,
                        T* xyz_grad, int accumulate, hipStream_t s) {
    const Plan& plan = planned.plan;
    const Launch& lanes = planned.lanes;
    if (planned.use_lanes) {
        auto launch = [&](auto kernel) -> hipError_t {
            if (lanes.lds_bytes > 64u * 1024u) {
                unsigned unused = 0;
                hipError_t err = kernel_facts(reinterpret_cast<const void*>(kernel), lanes.threads,
                                              lanes.lds_bytes, &unused);
                if (err != hipSuccess) return err;
            }
            hipLaunchKernelGGL(kernel, dim3(lanes.workgroups), dim3(lanes.threads), lanes.lds_bytes, s,
                               lanes.g, xyz, sph_grad, xyz_grad, accumulate);
            return hipGetLastError();
        };
        if (!planned.lane_groups) {
            if (lanes.threads > 512) {
                return normalized ? launch(vjp_lanes_kernel<T, true, 1024>) : launch(vjp_lanes_kernel<T, false, 1024>);
            }
            return normalized ? launch(vjp_lanes_kernel<T, true>) : launch(vjp_lanes_kernel<T, false>);
        }
        return normalized ? launch(vjp_groups_kernel<T, true>) : launch(vjp_groups_kernel<T, false>);
    }
    if (plan.closed_only) {
        return normalized ? dispatch_vjp_closed<T, true>(plan.closed, l_max, xyz, sph_grad, xyz_grad, accumulate, s)
                          : dispatch_vjp_closed<T, false>(plan.closed, l_max, xyz, sph_grad, xyz_grad, accumulate, s);
    }
    return normalized ? launch_vjp_recursion<T, true>(plan, xyz, sph_grad, xyz_grad, accumulate, s)
                      : launch_vjp_recursion<T, false>(plan, xyz, sph_grad, xyz_grad, accumulate, s);
}

template <typename T> hipError_t upload_vjp_tables(const HostTables& t) { return upload_tables<T>(t, nullptr, nullptr); }

} // namespace sphx

#endif
