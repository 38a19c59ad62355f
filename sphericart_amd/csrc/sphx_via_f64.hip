// float arrays evaluated in float64 (sphx_forward_f32_via_f64*): the conversion kernels, the library's static
// scratch array and the entry points.

#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "sphx_runtime.hpp"

namespace sphx {

// ---------------------------------------------------------------------------
// float32 arrays evaluated in float64. In float32 the reference's prefactors
// and Q_l^l = (2l-1)!! leave the range of the type from l = 29 (NaN and inf in
// the outputs) and high-|m| entries come out as exact zeros from l of about 20
// (sphericart/include/templates.hpp:54-97 evaluated in float). This path, which
// a caller must ask for, evaluates in float64 and rounds every result once:
// beyond the closed forms in one launch of the recursion kernel's mixed variant
// (forward_wide_on), else by widening xyz, running the float64 kernels into a
// workspace and narrowing the rows (below).
// ---------------------------------------------------------------------------
constexpr unsigned kConvertThreads = 256;

__global__ __launch_bounds__(kConvertThreads) void widen_kernel(const float* __restrict__ in,
                                                               double* __restrict__ out,
                                                               unsigned long long count) {
    const unsigned long long stride = static_cast<unsigned long long>(gridDim.x) * kConvertThreads;
    for (unsigned long long i = static_cast<unsigned long long>(blockIdx.x) * kConvertThreads + threadIdx.x;
         i < count; i += stride) {
        out[i] = static_cast<double>(in[i]);
    }
}

__global__ __launch_bounds__(kConvertThreads) void narrow_kernel(const double* __restrict__ in,
                                                                float* __restrict__ out,
                                                                unsigned long long count) {
    const unsigned long long stride = static_cast<unsigned long long>(gridDim.x) * kConvertThreads;
    for (unsigned long long i = static_cast<unsigned long long>(blockIdx.x) * kConvertThreads + threadIdx.x;
         i < count; i += stride) {
        out[i] = static_cast<float>(in[i]); // round to nearest even, overflow to infinity
    }
}

static unsigned convert_blocks(unsigned long long count) {
    const unsigned long long want = (count + kConvertThreads - 1) / kConvertThreads;
    return static_cast<unsigned>(want < 16384ull ? (want ? want : 1ull) : 16384ull);
}

// float64 bytes one point needs in the workspace: its coordinates and its rows
static size_t via_f64_bytes_per_point(int l_max, int mode) {
    const size_t ny = static_cast<size_t>(l_max + 1) * (l_max + 1);
    return sizeof(double) * (3 + ny * components_of(mode));
}

// The library's own scratch memory for sphx_forward_f32_via_f64_static: callers that must not
// allocate (HIP graph capture, serving loops, harnesses that forbid it) get the float64 rows of one
// call staged here. Every device the library runs on holds its own copy of the array, at its own
// address, until the process ends; device_state(device).scratch is that address, asked from the runtime once
// per device (ensure_device_ready keeps it in the device's state). In host code the array's name is only a handle for that
// question, never an address to hand to a kernel.
constexpr size_t kScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// with the device current; called once per device by ensure_device_ready
int find_scratch(void** address) {
    void* ptr = nullptr;
    SPHX_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr) return fail(SPHX_ERR_HIP, "hipGetSymbolAddress returned no address for the scratch array");
    *address = ptr;
    return SPHX_OK;
}

static int check_via_f64_arguments(const float* xyz, int l_max, int mode, const float* sph,
                                   const float* dsph, const float* ddsph) {
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (l_max > SPHX_TABLE_LMAX) {
        return fail(SPHX_ERR_UNSUPPORTED, "l_max = " + std::to_string(l_max) +
                                              " exceeds the device prefactor tables (" +
                                              std::to_string(SPHX_TABLE_LMAX) + ")");
    }
    if (xyz == nullptr) return fail(SPHX_ERR_ARGUMENT, "xyz is a null pointer");
    if (sph == nullptr) return fail(SPHX_ERR_ARGUMENT, "sph is a null pointer");
    if (mode >= 1 && dsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "dsph is a null pointer");
    if (mode >= 2 && ddsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "ddsph is a null pointer");
    return SPHX_OK;
}

// The points in chunks of as many as the workspace holds: widen, evaluate in float64, narrow.
// `device` is current. Enqueues only.
static int via_f64_chunks(int device, const float* xyz, size_t n_samples, int l_max, int normalized,
                          int mode, float* sph, float* dsph, float* ddsph, void* workspace,
                          size_t workspace_bytes, void* stream) {
    const size_t per_point = via_f64_bytes_per_point(l_max, mode);
    const size_t ny = static_cast<size_t>(l_max + 1) * (l_max + 1);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    size_t chunk = workspace_bytes / per_point;
    if (chunk == 0) {
        return fail(SPHX_ERR_ARGUMENT, "the workspace holds no point: " + std::to_string(per_point) +
                                           " bytes are needed per point");
    }
    if ((reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
        return fail(SPHX_ERR_ARGUMENT, "the workspace must be aligned to 16 bytes");
    }
    if (chunk >= n_samples) {
        chunk = n_samples; // one chunk
    } else if (chunk >= 64) {
        chunk &= ~size_t(63); // whole tiles of the closed-form kernels
    }
    // workspace layout for a chunk of c points: sph[c][ny], dsph[c][3][ny], ddsph[c][9][ny], xyz[c][3]
    double* w_sph = static_cast<double*>(workspace);
    double* w_dsph = w_sph + chunk * ny;
    double* w_ddsph = w_dsph + (mode >= 1 ? chunk * 3 * ny : 0);
    double* w_xyz = w_ddsph + (mode >= 2 ? chunk * 9 * ny : 0);
    for (size_t first = 0; first < n_samples; first += chunk) {
        const size_t count = n_samples - first < chunk ? n_samples - first : chunk;
        hipLaunchKernelGGL(widen_kernel, dim3(convert_blocks(count * 3)), dim3(kConvertThreads), 0, s,
                           xyz + first * 3, w_xyz, static_cast<unsigned long long>(count * 3));
        const int status = forward_on<double>(device, w_xyz, count, l_max, normalized, mode, w_sph,
                                              mode >= 1 ? w_dsph : nullptr, mode >= 2 ? w_ddsph : nullptr,
                                              stream);
        if (status != SPHX_OK) return status;
        hipLaunchKernelGGL(narrow_kernel, dim3(convert_blocks(count * ny)), dim3(kConvertThreads), 0, s,
                           w_sph, sph + first * ny, static_cast<unsigned long long>(count * ny));
        if (mode >= 1) {
            hipLaunchKernelGGL(narrow_kernel, dim3(convert_blocks(count * 3 * ny)), dim3(kConvertThreads), 0,
                               s, w_dsph, dsph + first * 3 * ny, static_cast<unsigned long long>(count * 3 * ny));
        }
        if (mode >= 2) {
            hipLaunchKernelGGL(narrow_kernel, dim3(convert_blocks(count * 9 * ny)), dim3(kConvertThreads), 0,
                               s, w_ddsph, ddsph + first * 9 * ny, static_cast<unsigned long long>(count * 9 * ny));
        }
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
        }
    }
    return SPHX_OK;
}

static int forward_f32_via_f64(const float* xyz, size_t n_samples, int l_max, int normalized, int mode,
                               float* sph, float* dsph, float* ddsph, void* workspace,
                               size_t workspace_bytes, void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
    int status = check_via_f64_arguments(xyz, l_max, mode, sph, dsph, ddsph);
    if (status != SPHX_OK) return status;

    hipPointerAttribute_t attr;
    SPHX_HIP(hipPointerGetAttributes(&attr, xyz));
    int current = 0;
    SPHX_HIP(hipGetDevice(&current));
    const int device = attr.device;
    if (device != current) SPHX_HIP(hipSetDevice(device));

    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    void* owned = nullptr;
    // Beyond the closed forms the recursion kernel does it all in one launch: it reads the float
    // coordinates, computes in float64 and stages float rows. No workspace is touched then.
    bool fused = false;
    status = forward_wide_on(device, xyz, n_samples, l_max, normalized, mode, sph, dsph, ddsph, stream, &fused);
    if (status == SPHX_OK && !fused && workspace == nullptr) {
        // No workspace given: one of our own for at most 256 MiB worth of points at a time, taken
        // from and returned to the device's memory pool in stream order, so that the call still
        // only enqueues (an allocation that waits for the device would stall the caller).
        const size_t per_point = via_f64_bytes_per_point(l_max, mode);
        size_t points = (size_t(256) << 20) / per_point;
        if (points < 64) points = 64;
        if (points > n_samples) points = n_samples;
        workspace_bytes = points * per_point;
        hipError_t e = hipMallocAsync(&owned, workspace_bytes, s);
        if (e != hipSuccess) {
            status = fail(SPHX_ERR_HIP, std::string("hipMallocAsync of the float64 workspace: ") + hipGetErrorString(e));
        }
        workspace = owned;
    }
    if (status == SPHX_OK && !fused) {
        status = via_f64_chunks(device, xyz, n_samples, l_max, normalized, mode, sph, dsph, ddsph, workspace,
                                workspace_bytes, stream);
    }
    if (owned != nullptr) {
        hipError_t e = hipFreeAsync(owned, s); // after the work enqueued above, in stream order
        if (e != hipSuccess && status == SPHX_OK) {
            status = fail(SPHX_ERR_HIP, std::string("hipFreeAsync: ") + hipGetErrorString(e));
        }
    }
    if (device != current) {
        hipError_t e = hipSetDevice(current);
        if (e != hipSuccess && status == SPHX_OK) {
            status = fail(SPHX_ERR_HIP, std::string("hipSetDevice: ") + hipGetErrorString(e));
        }
    }
    return status;
}

// The same without allocating anything. Beyond the closed forms the one launch of the mixed recursion kernel
// needs no workspace at all, and any number of points goes; below, the library's scratch array is the workspace
// for one chunk (widen, the float64 kernels, narrow: a fixed, short sequence of launches), and more points than
// it holds are refused.
static int forward_f32_via_f64_static(const float* xyz, size_t n_samples, int l_max, int normalized,
                                      int mode, float* sph, float* dsph, float* ddsph, void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
    int status = check_via_f64_arguments(xyz, l_max, mode, sph, dsph, ddsph);
    if (status != SPHX_OK) return status;
    return on_device_of(xyz, [&](int device) {
        bool fused = false;
        int done = forward_wide_on(device, xyz, n_samples, l_max, normalized, mode, sph, dsph, ddsph, stream, &fused);
        if (done != SPHX_OK || fused) return done;
        const size_t per_point = via_f64_bytes_per_point(l_max, mode);
        if (n_samples > kScratchBytes / per_point) {
            return fail(SPHX_ERR_UNSUPPORTED,
                        std::to_string(n_samples) + " points of " + std::to_string(per_point) +
                            " bytes each exceed the library's scratch memory of " + std::to_string(kScratchBytes) +
                            " bytes: at most " + std::to_string(kScratchBytes / per_point) +
                            " points of this shape per call");
        }
        // (forward_wide_on has made the device ready, which finds its copy of the scratch array.)
        // Every number of the part of the scratch this call uses is written (widen_kernel, the
        // float64 kernels) before it is read (the kernels, narrow_kernel), whatever the last
        // call left there: nothing has to be cleared.
        return via_f64_chunks(device, xyz, n_samples, l_max, normalized, mode, sph, dsph, ddsph,
                              device_state(device).scratch, kScratchBytes, stream);
    });
}

} // namespace sphx

extern "C" {

int sphx_forward_f32_via_f64(const float* xyz, size_t n_samples, int l_max, int normalized,
                             int derivatives, float* sph, float* dsph, float* ddsph, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return sphx::forward_f32_via_f64(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph,
                                     workspace, workspace_bytes, stream);
}

int sphx_forward_f32_via_f64_static(const float* xyz, size_t n_samples, int l_max, int normalized,
                                    int derivatives, float* sph, float* dsph, float* ddsph, void* stream) {
    return sphx::forward_f32_via_f64_static(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph,
                                            stream);
}

size_t sphx_forward_f32_via_f64_static_capacity(int l_max, int derivatives) {
    if (l_max < 0 || l_max > SPHX_TABLE_LMAX || derivatives < 0 || derivatives > 2) return 0;
    return sphx::kScratchBytes / sphx::via_f64_bytes_per_point(l_max, derivatives);
}

size_t sphx_forward_f32_via_f64_workspace(size_t n_samples, int l_max, int derivatives) {
    if (l_max < 0 || derivatives < 0 || derivatives > 2) return 0;
    return n_samples * sphx::via_f64_bytes_per_point(l_max, derivatives);
}

} // extern "C"
