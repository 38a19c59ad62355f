// The C-ABI launch layer declared in include/sphx_launch.h: device set-up, the plans of recent calls and the
// entry points. Host code; the kernels are instantiated in sphx_forward_*.hip, sphx_wide_*.hip, sphx_vjp_*.hip,
// sphx_pairs.hip and sphx_backward.hip, the planner is sphx_plan.cpp.
//
// Work decomposition. The outputs of consecutive points are consecutive in every output array, so a workgroup
// takes a *tile* of S consecutive points, builds the tile's slice of sph / dsph / ddsph in LDS in exactly the
// HBM layout, and then streams the three slices out with contiguous 16-byte stores: every 128-byte line of the
// outputs is written once, in full, by neighbouring lanes. Inside a tile
//
//   * l <= H (H = 6, or 1 when second derivatives are asked for: the split of the reference CPU classes,
//     sphericart/src/sphericart.cpp:45-92) is evaluated in closed form, one point per lane, in registers;
//   * every l > H is one independent job per (point, l) pair (the reference makes channels independent on
//     purpose, sphericart/include/templates_core.hpp:77-80), so the lanes of the workgroup run the Q_l^m
//     recursions of different l side by side.
//
// The prefactor tables are computed on the host (sphx_tables.cpp) with the reference's recurrences and kept in
// constant memory; they depend on (l, m) only, so one table up to SPHX_TABLE_LMAX serves every l_max.

#include "sphx_runtime.hpp"

#include <atomic>
#include <cstdio>
#include <mutex>
#include <vector>

namespace sphx {

// ---- devices ---------------------------------------------------------------------------------------------

static std::mutex g_init_mutex;
static std::atomic<bool> g_ready[kMaxDevices];
static DeviceState g_devices[kMaxDevices];

const DeviceState& device_state(int device) { return g_devices[device]; }

static int prepare_device(int device) {
    DeviceState fresh;
    const HostTables& t = host_tables();
    SPHX_HIP((upload_forward_tables<float, 0>(t, nullptr, nullptr)));
    SPHX_HIP((upload_forward_tables<float, 1>(t, &fresh.F32, &fresh.Q32)));
    SPHX_HIP((upload_forward_tables<float, 2>(t, nullptr, nullptr)));
    SPHX_HIP((upload_forward_tables<double, 0>(t, nullptr, nullptr)));
    SPHX_HIP((upload_forward_tables<double, 1>(t, &fresh.F64, &fresh.Q64)));
    SPHX_HIP((upload_forward_tables<double, 2>(t, nullptr, nullptr)));
    SPHX_HIP(upload_wide_tables<0>(t));
    SPHX_HIP(upload_wide_tables<1>(t));
    SPHX_HIP(upload_wide_tables<2>(t));
    SPHX_HIP(upload_vjp_tables<float>(t));
    SPHX_HIP(upload_vjp_tables<double>(t));
    SPHX_HIP(hipDeviceGetAttribute(&fresh.lds_limit, hipDeviceAttributeMaxSharedMemoryPerBlock, device));
    SPHX_HIP(hipDeviceGetAttribute(&fresh.compute_units, hipDeviceAttributeMultiprocessorCount, device));
    // The kernels deal their workgroups to eight XCDs (`blockIdx.x & 7`): on a device partitioned
    // otherwise the results would still be right but every XCD would write all over the outputs.
    // Said once, not enforced; a runtime that does not know the attribute is left alone.
    int xcds = 0;
    if (hipDeviceGetAttribute(&xcds, hipDeviceAttributeNumberOfXccs, device) != hipSuccess) {
        (void)hipGetLastError();
    } else if (xcds != 8 && xcds > 0) {
        std::fprintf(stderr,
                     "sphericart_amd: device %d reports %d XCDs; the kernels' workgroup order is laid out "
                     "for the 8 XCDs of an MI355X in SPX mode and will be slower here\n",
                     device, xcds);
    }
    const int status = find_scratch(&fresh.scratch);
    if (status != SPHX_OK) return status;
    g_devices[device] = fresh;
    return SPHX_OK;
}

int ensure_device_ready(int device) {
    if (device < 0 || device >= kMaxDevices) {
        return fail(SPHX_ERR_ARGUMENT, "device ordinal out of range");
    }
    // the steady state: one load, no lock
    if (g_ready[device].load(std::memory_order_acquire)) return SPHX_OK;
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_ready[device].load(std::memory_order_relaxed)) return SPHX_OK;
    const int status = prepare_device(device);
    if (status == SPHX_OK) g_ready[device].store(true, std::memory_order_release);
    return status;
}

// ---- kernels ---------------------------------------------------------------------------------------------

struct KernelFacts {
    int device;
    const void* kernel;
    unsigned lds_bytes;
    unsigned resident_workgroups; // on the whole device, a multiple of 8; 0 = unknown
};
static std::mutex g_facts_mutex;
static std::vector<KernelFacts> g_facts;
// what this thread asked last: a steady stream of equal calls takes no lock
static thread_local KernelFacts t_last_facts = {-1, nullptr, 0u, 0u};

hipError_t kernel_facts(const void* kernel, unsigned threads, unsigned lds_bytes, unsigned* resident_workgroups) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    if (t_last_facts.kernel == kernel && t_last_facts.device == device && t_last_facts.lds_bytes == lds_bytes) {
        *resident_workgroups = t_last_facts.resident_workgroups;
        return hipSuccess;
    }
    {
        std::lock_guard<std::mutex> lock(g_facts_mutex);
        for (const KernelFacts& f : g_facts) {
            if (f.device == device && f.kernel == kernel && f.lds_bytes == lds_bytes) {
                t_last_facts = f;
                *resident_workgroups = f.resident_workgroups;
                return hipSuccess;
            }
        }
    }
    const bool known = device >= 0 && device < kMaxDevices && g_ready[device].load(std::memory_order_acquire);
    if (lds_bytes > 64u * 1024u) {
        // the limit of the device, not of this launch: the attribute belongs to the kernel, and
        // a later launch with less must not lower it for one with more that is already cached
        int limit = known ? g_devices[device].lds_limit : 0;
        if (limit < static_cast<int>(lds_bytes)) limit = static_cast<int>(lds_bytes);
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, limit);
        if (e != hipSuccess) return e;
    }
    KernelFacts fresh{device, kernel, lds_bytes, 0u};
    int per_cu = 0;
    const int cus = known ? g_devices[device].compute_units : 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, static_cast<int>(threads), lds_bytes) ==
            hipSuccess &&
        per_cu > 0 && cus > 0) {
        fresh.resident_workgroups = (static_cast<unsigned>(per_cu) * static_cast<unsigned>(cus)) & ~7u;
    } else {
        (void)hipGetLastError();
    }
    std::lock_guard<std::mutex> lock(g_facts_mutex);
    g_facts.push_back(fresh);
    t_last_facts = fresh;
    *resident_workgroups = fresh.resident_workgroups;
    return hipSuccess;
}

// ---- the plans of recent calls ---------------------------------------------------------------------------
// Planning is a few hundred host instructions. A thread keeps the plans of the shapes it called last in a table
// indexed by a hash of the shape: a call whose shape is there compares one key and plans nothing.

constexpr unsigned kPlannedCalls = 64; // a power of two
static thread_local PlannedCall t_planned[kPlannedCalls];
static thread_local unsigned t_generation = 0;

PlannedCall* planned_call(int kind, size_t n_samples, int l_max, int mode, int elem, int normalized, int device,
                          bool* fresh) {
    t_generation = refresh_switches();
    unsigned long long h = static_cast<unsigned long long>(n_samples) * 0x9E3779B97F4A7C15ull;
    h ^= static_cast<unsigned long long>((((((kind * 3 + mode) * 2 + normalized) * 16 + elem) * 128 + l_max) * 64 +
                                          device)) * 0xD1342543DE82EF95ull;
    PlannedCall* c = &t_planned[(h >> 40) & (kPlannedCalls - 1u)];
    if (c->generation == t_generation && c->kind == kind && c->n_samples == n_samples && c->l_max == l_max &&
        c->mode == mode && c->elem == elem && c->normalized == normalized && c->device == device) {
        *fresh = false;
        return c;
    }
    c->generation = 0;
    c->kind = kind;
    c->n_samples = n_samples;
    c->l_max = l_max;
    c->mode = mode;
    c->elem = elem;
    c->normalized = normalized;
    c->device = device;
    c->wide = false;
    *fresh = true;
    return c;
}

void keep(PlannedCall* call) { call->generation = t_generation; }

// ---- forward ---------------------------------------------------------------------------------------------

template <typename T>
int forward_on(int device, const T* xyz, size_t n_samples, int l_max, int normalized, int mode, T* sph, T* dsph,
               T* ddsph, void* stream) {
    int status = ensure_device_ready(device);
    if (status != SPHX_OK) return status;
    const DeviceState& dev = g_devices[device];
    bool fresh = false;
    PlannedCall* call = planned_call(0, n_samples, l_max, mode, sizeof(T), normalized != 0, device, &fresh);
    if (fresh) {
        status = make_plan(n_samples, l_max, mode, sizeof(T), dev.lds_limit, dev.compute_units, &call->plan, true,
                           normalized != 0);
        if (status != SPHX_OK) return status;
        keep(call);
    }
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool norm = normalized != 0;
    const hipError_t e = mode == 0   ? dispatch_forward<T, 0>(call->plan, dev, norm, xyz, sph, dsph, ddsph, s)
                         : mode == 1 ? dispatch_forward<T, 1>(call->plan, dev, norm, xyz, sph, dsph, ddsph, s)
                                     : dispatch_forward<T, 2>(call->plan, dev, norm, xyz, sph, dsph, ddsph, s);
    if (e != hipSuccess) {
        return fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
    }
    return SPHX_OK;
}
template int forward_on<float>(int, const float*, size_t, int, int, int, float*, float*, float*, void*);
template int forward_on<double>(int, const double*, size_t, int, int, int, double*, double*, double*, void*);

int forward_wide_on(int device, const float* xyz, size_t n_samples, int l_max, int normalized, int mode,
                    float* sph, float* dsph, float* ddsph, void* stream, bool* taken) {
    *taken = false;
    int status = ensure_device_ready(device);
    if (status != SPHX_OK) return status;
    const DeviceState& dev = g_devices[device];
    bool fresh = false;
    PlannedCall* call = planned_call(2, n_samples, l_max, mode, 8, normalized != 0, device, &fresh);
    if (fresh) {
        call->wide = make_wide_plan(n_samples, l_max, mode, dev.lds_limit, dev.compute_units, &call->plan,
                                    normalized != 0);
        keep(call);
    }
    if (!call->wide) return SPHX_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool norm = normalized != 0;
    const hipError_t e = mode == 0   ? dispatch_wide<0>(call->plan, norm, xyz, sph, dsph, ddsph, s)
                         : mode == 1 ? dispatch_wide<1>(call->plan, norm, xyz, sph, dsph, ddsph, s)
                                     : dispatch_wide<2>(call->plan, norm, xyz, sph, dsph, ddsph, s);
    if (e != hipSuccess) {
        return fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
    }
    *taken = true;
    return SPHX_OK;
}

template <typename T>
static int forward(const T* xyz, size_t n_samples, int l_max, int normalized, int mode, T* sph, T* dsph, T* ddsph,
                   void* stream) {
    t_error.clear();
    if (n_samples == 0) {
        return SPHX_OK;
    }
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (xyz == nullptr) return fail(SPHX_ERR_ARGUMENT, "xyz is a null pointer");
    if (sph == nullptr) return fail(SPHX_ERR_ARGUMENT, "sph is a null pointer");
    if (mode >= 1 && dsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "dsph is a null pointer");
    if (mode >= 2 && ddsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "ddsph is a null pointer");
    return on_device_of(xyz, [&](int device) {
        return forward_on<T>(device, xyz, n_samples, l_max, normalized, mode, sph, dsph, ddsph, stream);
    });
}

// ---- the fused product -----------------------------------------------------------------------------------

template <typename T>
static int vjp(const T* xyz, const T* sph_grad, size_t n_samples, int l_max, int normalized, T* xyz_grad,
               int accumulate, void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (xyz == nullptr || sph_grad == nullptr || xyz_grad == nullptr) {
        return fail(SPHX_ERR_ARGUMENT, "null pointer passed to the vector-Jacobian product");
    }
    if ((n_samples + 63) / 64 > 0x7fffffffull) {
        return fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    }
    return on_device_of(xyz, [&](int device) {
        int status = ensure_device_ready(device);
        if (status != SPHX_OK) return status;
        if (l_max > SPHX_TABLE_LMAX) {
            return fail(SPHX_ERR_UNSUPPORTED, "l_max = " + std::to_string(l_max) +
                                                  " exceeds the device prefactor tables (" +
                                                  std::to_string(SPHX_TABLE_LMAX) + ")");
        }
        const DeviceState& dev = g_devices[device];
        bool fresh = false;
        PlannedCall* call = planned_call(1, n_samples, l_max, 1, sizeof(T), normalized != 0, device, &fresh);
        if (fresh) {
            status = make_vjp_plan(n_samples, l_max, sizeof(T), dev.lds_limit, dev.compute_units, &call->vjp);
            if (status != SPHX_OK) return status;
            keep(call);
        }
        const hipError_t e = dispatch_vjp<T>(call->vjp, l_max, normalized != 0, xyz, sph_grad, xyz_grad, accumulate,
                                             reinterpret_cast<hipStream_t>(stream));
        if (e != hipSuccess) {
            return fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
        }
        return static_cast<int>(SPHX_OK);
    });
}

// what the device is like for a plan that is only asked about; an MI355X where there is none
static void device_for_planning(int* lds, int* cus) {
    int device = 0;
    *lds = 160 * 1024;
    *cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, device) == hipSuccess && v > 0) *lds = v;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) *cus = v;
    } else {
        (void)hipGetLastError();
    }
}

} // namespace sphx

extern "C" {

int sphx_forward_f32(const float* xyz, size_t n_samples, int l_max, int normalized, int derivatives, float* sph,
                     float* dsph, float* ddsph, void* stream) {
    return sphx::forward<float>(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph, stream);
}

int sphx_forward_f64(const double* xyz, size_t n_samples, int l_max, int normalized, int derivatives, double* sph,
                     double* dsph, double* ddsph, void* stream) {
    return sphx::forward<double>(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph, stream);
}

int sphx_vjp_f32(const float* xyz, const float* sph_grad, size_t n_samples, int l_max, int normalized,
                 float* xyz_grad, int accumulate, void* stream) {
    return sphx::vjp<float>(xyz, sph_grad, n_samples, l_max, normalized, xyz_grad, accumulate, stream);
}

int sphx_vjp_f64(const double* xyz, const double* sph_grad, size_t n_samples, int l_max, int normalized,
                 double* xyz_grad, int accumulate, void* stream) {
    return sphx::vjp<double>(xyz, sph_grad, n_samples, l_max, normalized, xyz_grad, accumulate, stream);
}

int sphx_device_count(void) {
    sphx::t_error.clear();
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        sphx::t_error = std::string("hipGetDeviceCount: ") + hipGetErrorString(e);
        return -1;
    }
    return n;
}

const char* sphx_last_error(void) { return sphx::t_error.c_str(); }

int sphx_plan(size_t n_samples, int l_max, int derivatives, int is_f64, int* tile_samples, int* threads,
              int* lds_bytes, int* workgroups) {
    sphx::t_error.clear();
    int lds = 0, cus = 0;
    sphx::device_for_planning(&lds, &cus);
    sphx::Plan plan;
    (void)sphx::refresh_switches();
    const int status = sphx::make_plan(n_samples ? n_samples : 1, l_max, derivatives,
                                       is_f64 ? sizeof(double) : sizeof(float), lds, cus, &plan);
    if (status != SPHX_OK) return status;
    if (plan.pairs) {
        if (tile_samples) *tile_samples = static_cast<int>(plan.pairs_launch.g.tile);
        if (threads) *threads = static_cast<int>(plan.pairs_launch.threads);
        if (lds_bytes) *lds_bytes = static_cast<int>(plan.pairs_launch.lds_bytes);
        if (workgroups) *workgroups = static_cast<int>(plan.pairs_launch.workgroups);
        return SPHX_OK;
    }
    const sphx::Launch& main = plan.closed_only || plan.lanes ? plan.closed : plan.rec;
    if (tile_samples) *tile_samples = main.g.tile;
    if (threads) *threads = static_cast<int>(main.threads);
    if (lds_bytes) *lds_bytes = static_cast<int>(main.lds_bytes);
    if (workgroups) *workgroups = static_cast<int>(main.workgroups);
    return SPHX_OK;
}

int sphx_describe_plan(size_t n_samples, int l_max, int derivatives, int is_f64, int normalized, char* out,
                       size_t capacity) {
    sphx::t_error.clear();
    if (out == nullptr || capacity == 0) return sphx::fail(SPHX_ERR_ARGUMENT, "no room for the description");
    int lds = 0, cus = 0;
    sphx::device_for_planning(&lds, &cus);
    sphx::Plan plan;
    (void)sphx::refresh_switches();
    const int status = sphx::make_plan(n_samples ? n_samples : 1, l_max, derivatives,
                                       is_f64 ? sizeof(double) : sizeof(float), lds, cus, &plan, true, normalized != 0);
    if (status != SPHX_OK) return status;
    std::snprintf(out, capacity, "%s", sphx::describe(plan, l_max, derivatives, is_f64 != 0, normalized != 0).c_str());
    return SPHX_OK;
}

int sphx_set_switch(const char* name, int value) {
    sphx::t_error.clear();
    return sphx::set_switch(name, value);
}

void sphx_reset_switches(void) { sphx::reset_switches(); }

} // extern "C"
