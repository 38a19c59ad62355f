// Host side of the launch layer that every translation unit with kernels shares: the state of a device (tables
// uploaded, LDS size, CUs), what the runtime says about a kernel, the plans of recent calls. The kernels are
// instantiated in translation units of their own (sphx_forward_*.hip, sphx_wide_*.hip, sphx_vjp_*.hip), one per
// arithmetic type and set of derivatives, so that they compile side by side; what they export is declared here.
#ifndef SPHX_RUNTIME_HPP
#define SPHX_RUNTIME_HPP

#include <hip/hip_runtime.h>

#include <string>

#include "../../include/sphx_launch.h"
#include "sphx_plan.hpp"
#include "sphx_tables.hpp"

namespace sphx {

#define SPHX_HIP(call)                                                                            \
    do {                                                                                          \
        hipError_t status_ = (call);                                                              \
        if (status_ != hipSuccess) {                                                              \
            return fail(SPHX_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(status_));    \
        }                                                                                         \
    } while (0)

constexpr int kMaxDevices = 64;

struct DeviceState {
    int lds_limit = 0;     // bytes of LDS a workgroup may have
    int compute_units = 0;
    // the constant tables as pairs_kernel takes them, by pointer
    const float *F32 = nullptr, *Q32 = nullptr;
    const double *F64 = nullptr, *Q64 = nullptr;
    void* scratch = nullptr; // the library's static scratch array on this device (sphx_via_f64.hip)
};

// Uploads the tables to every translation unit's constant memory on `device` (current) the first time, and
// asks the device what the planner needs to know. After SPHX_OK device_state(device) is filled in.
int ensure_device_ready(int device);
const DeviceState& device_state(int device);

// Raises the kernel's dynamic LDS limit if needed and returns how many workgroups of `threads` threads are
// resident on the current device at once (0 if the runtime would not tell). Asked from the runtime once per
// (device, kernel, LDS size): the calls take microseconds each, the whole budget of a small evaluation.
hipError_t kernel_facts(const void* kernel, unsigned threads, unsigned lds_bytes, unsigned* resident_workgroups);

// What a call of a given shape launches, kept per thread so that a steady stream of equal calls plans once.
struct PlannedCall {
    // key
    unsigned generation = 0; // of the overrides; 0 = empty slot
    int kind = 0;            // 0: forward, 1: fused product, 2: float arrays evaluated in float64
    size_t n_samples = 0;
    int l_max = 0, mode = 0, elem = 0, normalized = 0, device = 0;
    // what was planned
    Plan plan;         // kinds 0 and 2
    VjpPlan vjp;       // kind 1
    bool wide = false; // kind 2: the recursion kernel covers this shape
};
// The slot for this shape; `*fresh` says that it has yet to be planned (by the caller, who then calls keep();
// a plan that failed leaves the slot empty).
PlannedCall* planned_call(int kind, size_t n_samples, int l_max, int mode, int elem, int normalized, int device,
                          bool* fresh);
void keep(PlannedCall* call);

// Runs `body(device)` with the device that owns `pointer` current, and restores the caller's device.
template <typename Body> int on_device_of(const void* pointer, Body body) {
    hipPointerAttribute_t attr;
    SPHX_HIP(hipPointerGetAttributes(&attr, pointer));
    int current = 0;
    SPHX_HIP(hipGetDevice(&current));
    const int device = attr.device;
    if (device != current) SPHX_HIP(hipSetDevice(device));
    int status = body(device);
    if (device != current) {
        hipError_t e = hipSetDevice(current);
        if (e != hipSuccess && status == SPHX_OK) {
            status = fail(SPHX_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
        }
    }
    return status;
}

// ---- what the translation units with kernels export -------------------------------------------------------
// (defined by explicit instantiation: sphx_dispatch.hpp, sphx_vjp_dispatch.hpp)

// The kernels of `plan` for arithmetic type T and MODE = 0 values, 1 with gradients, 2 with second derivatives.
template <typename T, int MODE>
hipError_t dispatch_forward(const Plan& plan, const DeviceState& device, bool normalized, const T* xyz, T* sph,
                            T* dsph, T* ddsph, hipStream_t stream);
// The same for float arrays evaluated in float64 (recursion_kernel with T = double, O = float).
template <int MODE>
hipError_t dispatch_wide(const Plan& plan, bool normalized, const float* xyz, float* sph, float* dsph, float* ddsph,
                         hipStream_t stream);
// The fused product xyz_grad = sum_k dsph * sph_grad.
template <typename T>
hipError_t dispatch_vjp(const VjpPlan& plan, int l_max, bool normalized, const T* xyz, const T* sph_grad,
                        T* xyz_grad, int accumulate, hipStream_t stream);
// Each of those translation units has the constant tables of its arithmetic type to itself; these fill them
// on the current device. `F` / `Q` (may be null) receive the device addresses.
template <typename T, int MODE> hipError_t upload_forward_tables(const HostTables& t, const T** F, const T** Q);
template <int MODE> hipError_t upload_wide_tables(const HostTables& t);
template <typename T> hipError_t upload_vjp_tables(const HostTables& t);

// The evaluation proper on `device`, which is current (sphx_forward_*; the float64 one also serves the float
// arrays that go through a float64 workspace).
template <typename T>
int forward_on(int device, const T* xyz, size_t n_samples, int l_max, int normalized, int mode, T* sph, T* dsph,
               T* ddsph, void* stream);
// float arrays in one launch of the mixed recursion kernel; *taken = false: not a shape for it, nothing enqueued.
int forward_wide_on(int device, const float* xyz, size_t n_samples, int l_max, int normalized, int mode,
                    float* sph, float* dsph, float* ddsph, void* stream, bool* taken);
// with `device` current: the address of the static scratch array on it (sphx_via_f64.hip)
int find_scratch(void** address);

} // namespace sphx

#endif
