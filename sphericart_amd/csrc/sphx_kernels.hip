// HIP kernels (gfx950) and the C-ABI launch layer declared in
// include/sphx_launch.h.
//
// Work decomposition. The outputs of consecutive points are consecutive in
// every output array, so a workgroup takes a *tile* of S consecutive points,
// builds the tile's slice of sph / dsph / ddsph in LDS in exactly the HBM
// layout, and then streams the three slices out with contiguous 16-byte
// stores: every 128-byte line of the outputs is written once, in full, by
// neighbouring lanes. Inside a tile
//
//   * l <= H (H = 6, or 1 when second derivatives are asked for: the split of
//     the reference CPU classes, sphericart/src/sphericart.cpp:45-92) is
//     evaluated in closed form, one point per lane, in registers;
//   * every l > H is one independent job per (point, l) pair
//     (the reference makes channels independent on purpose,
//     sphericart/include/templates_core.hpp:77-80), so the lanes of the
//     workgroup run the Q_l^m recursions of different l side by side.
//
// `closed_form_kernel` is the all-closed-form case (l_max <= 6 without second
// derivatives, l_max <= 1 with): one wave, one point per lane, 64 points per
// tile. `recursion_kernel` is the general case; its workgroups are persistent
// and walk over tiles so that the prefactor tables are fetched once.
//
// The prefactor tables are computed on the host (sphx_tables.cpp) with the
// reference's recurrences and kept in constant memory; they depend on (l, m)
// only, so one table up to SPHX_TABLE_LMAX serves every l_max.

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "../../include/sphx_launch.h"
#include "sphx_device.hpp"
#include "sphx_tables.hpp"

namespace sphx {

constexpr int kTableEntries = (SPHX_TABLE_LMAX + 1) * (SPHX_TABLE_LMAX + 2) / 2;

__constant__ float kF32[kTableEntries];
__constant__ float kQ32[kTableEntries];
__constant__ double kF64[kTableEntries];
__constant__ double kQ64[kTableEntries];

template <typename T> __device__ __forceinline__ const T* table_F();
template <typename T> __device__ __forceinline__ const T* table_Q();
template <> __device__ __forceinline__ const float* table_F<float>() { return kF32; }
template <> __device__ __forceinline__ const float* table_Q<float>() { return kQ32; }
template <> __device__ __forceinline__ const double* table_F<double>() { return kF64; }
template <> __device__ __forceinline__ const double* table_Q<double>() { return kQ64; }

// Everything a kernel needs to know about the tiling; filled in on the host.
struct Tiling {
    unsigned long long n_samples;
    unsigned n_tiles;
    int l_max;
    int ny;          // (l_max + 1)^2
    int tile;        // points per tile (S)
    unsigned pad;    // spare LDS elements after each point's block (0 or 1)
    unsigned magic[3]; // ceil(2^32 / row) for row = ny, 3 ny, 9 ny
    // LDS carve-up, in elements of T from the start of dynamic LDS
    unsigned off_dsph, off_ddsph, off_F, off_Q, off_pts, off_jobs;
    // every l channel above the closed-form limit is cut into segments of `segment`
    // consecutive m; one point has `jobs_per_point` (channel, segment) jobs in all
    unsigned segment, jobs_per_point;
    // persistent-workgroup walk: workgroups of one XCD take consecutive tiles
    unsigned tiles_per_group;
};

extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];

// Output lines are written once and never read back by the kernel: store them with the
// non-temporal hint (measured 10-20 % faster than plain stores here).
#ifndef SPHX_STREAMING_STORES
#define SPHX_STREAMING_STORES true
#endif

// Stream the staged rows of `valid` consecutive points, the first of which is
// point number `first`, from LDS to the output arrays.
template <typename T, int MODE>
__device__ __forceinline__ void flush_run(const Tiling& g, T* lds, unsigned long long first,
                                          unsigned valid, T* sph, T* dsph, T* ddsph,
                                          unsigned tid, unsigned nthreads) {
    const unsigned ny = g.ny;
    copy_out<T, SPHX_STREAMING_STORES>(lds, sph + first * ny, valid * ny, ny, g.pad, g.magic[0], tid,
                                       nthreads);
    if constexpr (MODE >= 1) {
        copy_out<T, SPHX_STREAMING_STORES>(lds + g.off_dsph, dsph + first * 3 * ny, valid * 3 * ny,
                                           3 * ny, g.pad, g.magic[1], tid, nthreads);
    }
    if constexpr (MODE == 2) {
        copy_out<T, SPHX_STREAMING_STORES>(lds + g.off_ddsph, ddsph + first * 9 * ny, valid * 9 * ny,
                                           9 * ny, g.pad, g.magic[2], tid, nthreads);
    }
}

template <typename T, int MODE>
__device__ __forceinline__ Rows<T> rows_of(const Tiling& g, T* lds, unsigned s) {
    Rows<T> r;
    r.ny = g.ny;
    r.sph = lds + s * (g.ny + g.pad);
    r.dsph = MODE >= 1 ? lds + g.off_dsph + s * (3 * g.ny + g.pad) : nullptr;
    r.ddsph = MODE == 2 ? lds + g.off_ddsph + s * (9 * g.ny + g.pad) : nullptr;
    return r;
}

// ---------------------------------------------------------------------------
// l_max = H, everything in closed form. One wave per workgroup, one point per
// lane, 64 points per workgroup.
//
// The finished numbers of a point stay in the lane's VGPRs; LDS is only the
// transposition buffer between "one point per lane" and "consecutive addresses
// per lane". To keep many waves resident per CU (the register file, not LDS,
// then bounds the bytes in flight) the 64 points go through the buffer in
// PHASES passes of 64 / PHASES points each; the slice of every output array
// that a pass covers is still one contiguous run.
// ---------------------------------------------------------------------------
// Bytes of LDS one pass may use: 52 KB lets three workgroups share a CU. Measured on MI355X,
// l_max = 6 float32 with gradients runs fastest with a single pass (50 KB).
#ifndef SPHX_PHASE_LDS_BUDGET
#define SPHX_PHASE_LDS_BUDGET (52 * 1024)
#endif

__host__ __device__ constexpr unsigned closed_form_phases(unsigned elem, int mode, int H) {
    const unsigned ny = (H + 1) * (H + 1);
    const unsigned arrays = mode + 1;
    const unsigned mult = mode == 0 ? 1 : (mode == 1 ? 4 : 13);
    const unsigned per_point = (mult * ny + arrays * (ny % 2 == 0 ? 1u : 0u)) * elem;
    unsigned phases = 1;
    while (phases < 16 && (64 / phases) * per_point > SPHX_PHASE_LDS_BUDGET) {
        phases *= 2;
    }
    return phases;
}

template <typename T, int MODE, bool NORM, int H>
__global__ __launch_bounds__(64) void closed_form_kernel(Tiling g, const T* __restrict__ xyz,
                                                        T* __restrict__ sph, T* __restrict__ dsph,
                                                        T* __restrict__ ddsph) {
    constexpr unsigned PHASES = closed_form_phases(sizeof(T), MODE, H);
    constexpr unsigned PER = 64 / PHASES;
    constexpr unsigned NY = (H + 1) * (H + 1);
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    // Workgroups are handed to the 8 XCDs round-robin; give each XCD one contiguous stretch of
    // points, so that what one XCD writes at any moment is a compact window of each array
    // (measured: 6 % faster than the identity mapping).
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_group + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned long long first = static_cast<unsigned long long>(group) * 64;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < 64ull ? static_cast<unsigned>(left) : 64u;
    // the row length is a compile-time constant here: rebuild the geometry with it
    Tiling gc = g;
    gc.ny = NY;
    gc.tile = PER;
    gc.pad = (NY % 2 == 0) ? 1u : 0u;
    gc.magic[0] = static_cast<unsigned>(((1ull << 32) + NY - 1) / NY);
    gc.magic[1] = static_cast<unsigned>(((1ull << 32) + 3 * NY - 1) / (3 * NY));
    gc.magic[2] = static_cast<unsigned>(((1ull << 32) + 9 * NY - 1) / (9 * NY));

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
            const Rows<T> rows = rows_of<T, MODE>(gc, lds, tid - base);
#pragma unroll
            for (unsigned k = 0; k < NY; ++k) {
                put<T, MODE>(rows, k, E[k]);
            }
        }
        __syncthreads();
        const unsigned count = valid - base < PER ? valid - base : PER;
        flush_run<T, MODE>(gc, lds, first + base, count, sph, dsph, ddsph, tid, 64);
    }
}

// ---------------------------------------------------------------------------
// General case: closed form up to H, recursion above. 256 threads; wave 0
// hosts the per-point lanes, waves 1..3 the (point, l) jobs.
// ---------------------------------------------------------------------------
template <typename T, int MODE, bool NORM, int H>
__global__ __launch_bounds__(256) void recursion_kernel(Tiling g, const T* __restrict__ xyz,
                                                       T* __restrict__ sph, T* __restrict__ dsph,
                                                       T* __restrict__ ddsph) {
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned nthreads = blockDim.x;
    const int L = g.l_max;
    const unsigned S = g.tile;

    T* F = lds + g.off_F;
    T* Q = lds + g.off_Q;
    unsigned short* job_table = reinterpret_cast<unsigned short*>(lds + g.off_jobs);
    {
        const unsigned nq = (L + 1) * (L + 2) / 2;
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        for (unsigned i = tid; i < nq; i += nthreads) {
            F[i] = cF[i];
            Q[i] = cQ[i];
        }
        // (l, segment) pairs, top segments of all channels first, longest channels first:
        // neighbouring lanes then run loops of the same length
        if (tid == 0) {
            unsigned n = 0;
            for (unsigned seg = 0; seg * g.segment <= static_cast<unsigned>(L); ++seg) {
                for (int l = L; l > H; --l) {
                    if (seg * g.segment <= static_cast<unsigned>(l)) {
                        job_table[n++] = static_cast<unsigned short>((l << 8) | seg);
                    }
                }
            }
        }
    }

    // Workgroups are handed to the 8 XCDs round-robin; give each XCD one
    // contiguous stretch of tiles so that lines shared by neighbouring tiles
    // meet in one L2.
    const unsigned xcd = blockIdx.x & 7u;
    const unsigned lane_in_xcd = blockIdx.x >> 3;
    const unsigned groups_per_xcd = gridDim.x >> 3;
    const unsigned xcd_first = xcd * g.tiles_per_group;
    unsigned xcd_last = xcd_first + g.tiles_per_group;
    if (xcd_last > g.n_tiles) xcd_last = g.n_tiles;

    // Per-point data (normalised coordinates, c_m, s_m, 2(m+1)z) is double buffered: while the
    // recursion jobs of one tile run, wave 0 prepares the next tile, so that the LDS rows are
    // only held from the first staged entry to the end of the flush.
    const unsigned per_point_tables = 3 * (L + 1) + 8;
    auto tables_of = [&](unsigned parity, unsigned s) -> T* {
        return lds + g.off_pts + (parity * S + s) * per_point_tables;
    };
    auto prepare = [&](unsigned tile_idx, unsigned parity, T rx, T ry, T rz) {
        // templates.hpp:386-400 and :451-466 for point `tid` of the tile
        (void)tile_idx;
        T* rec = tables_of(parity, tid);
        Point<T> p;
        p.x = rx;
        p.y = ry;
        p.z = rz;
        p.x2 = p.x * p.x;
        p.y2 = p.y * p.y;
        p.z2 = p.z * p.z;
        p.ir = 0.0;
        if constexpr (NORM) {
            p.ir = 1 / root(p.x2 + p.y2 + p.z2);
            p.x *= p.ir;
            p.y *= p.ir;
            p.z *= p.ir;
            p.x2 = p.x * p.x;
            p.y2 = p.y * p.y;
            p.z2 = p.z * p.z;
        }
        rec[0] = p.x;
        rec[1] = p.y;
        rec[2] = p.z;
        rec[3] = p.x2;
        rec[4] = p.y2;
        rec[5] = p.z2;
        rec[6] = p.ir;
        azimuth_job<T>(p, L, rec + 8, rec + 8 + (L + 1), rec + 8 + 2 * (L + 1));
    };
    auto point_of = [&](const T* rec) {
        Point<T> q;
        q.x = rec[0];
        q.y = rec[1];
        q.z = rec[2];
        q.x2 = rec[3];
        q.y2 = rec[4];
        q.z2 = rec[5];
        q.ir = rec[6];
        return q;
    };
    auto valid_in = [&](unsigned tile_idx) -> unsigned {
        const unsigned long long first = static_cast<unsigned long long>(tile_idx) * S;
        const unsigned long long left = g.n_samples - first;
        return left < S ? static_cast<unsigned>(left) : S;
    };

    unsigned tile_idx = xcd_first + lane_in_xcd;
    unsigned parity = 0;
    if (tile_idx < xcd_last && tid < valid_in(tile_idx)) {
        const T* src = xyz + (static_cast<unsigned long long>(tile_idx) * S + tid) * 3;
        prepare(tile_idx, 0, src[0], src[1], src[2]);
    }

    for (; tile_idx < xcd_last; tile_idx += groups_per_xcd, parity ^= 1u) {
        const unsigned long long first = static_cast<unsigned long long>(tile_idx) * S;
        const unsigned valid = valid_in(tile_idx);
        const unsigned next_idx = tile_idx + groups_per_xcd;
        const unsigned next_valid = next_idx < xcd_last ? valid_in(next_idx) : 0u;

        __syncthreads(); // rows free again (previous flush done); this tile's point data in place

        if (tid < 64) {
            // fetch the next tile's coordinates now, use them after the closed-form work
            T nx = 0, ny_ = 0, nz = 0;
            if (tid < next_valid) {
                const T* src = xyz + (static_cast<unsigned long long>(next_idx) * S + tid) * 3;
                nx = src[0];
                ny_ = src[1];
                nz = src[2];
            }
            if (tid < valid) {
                const Point<T> p = point_of(tables_of(parity, tid));
                closed_form_job<T, MODE, NORM, H>(p, rows_of<T, MODE>(g, lds, tid));
            }
            if (tid < next_valid) {
                prepare(next_idx, parity ^ 1u, nx, ny_, nz);
            }
        } else {
            const unsigned jobs = valid * g.jobs_per_point;
            for (unsigned j = tid - 64; j < jobs; j += nthreads - 64) {
                const unsigned s = j % valid;
                const unsigned entry = job_table[j / valid];
                const int l = static_cast<int>(entry >> 8);
                const int m_hi = l - static_cast<int>((entry & 0xffu) * g.segment);
                const int m_lo = m_hi - static_cast<int>(g.segment) + 1 > 0
                                     ? m_hi - static_cast<int>(g.segment) + 1
                                     : 0;
                const T* rec = tables_of(parity, s);
                const Point<T> q = point_of(rec);
                const T rxy = q.x2 + q.y2;
                channel_job<T, MODE, NORM>(l, m_hi, m_lo, q, rxy, F, Q, rec + 8, rec + 8 + (L + 1),
                                           rec + 8 + 2 * (L + 1), rows_of<T, MODE>(g, lds, s));
            }
        }
        __syncthreads();
        flush_run<T, MODE>(g, lds, first, valid, sph, dsph, ddsph, tid, nthreads);
    }
}

// ---------------------------------------------------------------------------
// Host side of the launch layer
// ---------------------------------------------------------------------------

thread_local std::string t_error;

static int fail(int code, const std::string& what) {
    t_error = what;
    return code;
}

#define SPHX_HIP(call)                                                                            \
    do {                                                                                          \
        hipError_t status_ = (call);                                                              \
        if (status_ != hipSuccess) {                                                              \
            return fail(SPHX_ERR_HIP, std::string(#call) + ": " + hipGetErrorString(status_));    \
        }                                                                                         \
    } while (0)

constexpr int kMaxDevices = 64;
static std::mutex g_init_mutex;
static bool g_tables_ready[kMaxDevices] = {};
static int g_lds_limit[kMaxDevices] = {};
static int g_compute_units[kMaxDevices] = {};

// Upload the tables to the constant memory of `device` (current) once.
static int ensure_device_ready(int device) {
    if (device < 0 || device >= kMaxDevices) {
        return fail(SPHX_ERR_ARGUMENT, "device ordinal out of range");
    }
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_tables_ready[device]) {
        return SPHX_OK;
    }
    const HostTables& t = host_tables();
    const size_t n = kTableEntries;
    SPHX_HIP(hipMemcpyToSymbol(HIP_SYMBOL(kF32), t.f32.data(), n * sizeof(float)));
    SPHX_HIP(hipMemcpyToSymbol(HIP_SYMBOL(kQ32), t.f32.data() + n, n * sizeof(float)));
    SPHX_HIP(hipMemcpyToSymbol(HIP_SYMBOL(kF64), t.f64.data(), n * sizeof(double)));
    SPHX_HIP(hipMemcpyToSymbol(HIP_SYMBOL(kQ64), t.f64.data() + n, n * sizeof(double)));
    int lds = 0, cus = 0;
    SPHX_HIP(hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device));
    SPHX_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    g_lds_limit[device] = lds;
    g_compute_units[device] = cus;
    g_tables_ready[device] = true;
    return SPHX_OK;
}

static int env_int(const char* name, int fallback) {
    const char* v = std::getenv(name);
    if (!v || !*v) return fallback;
    return std::atoi(v);
}

struct Plan {
    Tiling g;
    bool closed_form;
    unsigned points_per_group;
    int threads;
    unsigned lds_bytes;
    unsigned workgroups;
};

static unsigned pow2_floor(unsigned v) {
    unsigned p = 1;
    while (2 * p <= v) p *= 2;
    return p;
}

// Choose tile size and LDS layout. `lds_limit` / `cus` describe the device.
static int make_plan(size_t n_samples, int l_max, int mode, size_t elem, int lds_limit, int cus,
                     Plan* plan) {
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (l_max > SPHX_TABLE_LMAX) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) + " exceeds the device prefactor tables (" +
                        std::to_string(SPHX_TABLE_LMAX) + ")");
    }
    Tiling& g = plan->g;
    std::memset(&g, 0, sizeof(g));
    const int hard_cap = mode == 2 ? 1 : 6;
    plan->closed_form = l_max <= hard_cap;
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned mult = mode == 0 ? 1 : (mode == 1 ? 4 : 13); // elements per point = mult * ny
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.pad = (ny % 2 == 0) ? 1u : 0u;
    const unsigned arrays = mode + 1;
    const unsigned row_elems = mult * ny + arrays * g.pad; // LDS elements per point

    unsigned S;         // points whose rows are staged in LDS at a time
    unsigned per_group; // points one workgroup handles before it moves on (or ends)
    if (plan->closed_form) {
        plan->threads = 64;
        per_group = 64;
        S = 64 / closed_form_phases(static_cast<unsigned>(elem), mode, l_max);
    } else {
        plan->threads = 256;
        const unsigned budget = static_cast<unsigned>(env_int("SPHX_TILE_LDS_BUDGET", 36 * 1024));
        const unsigned per_point = (row_elems + 2 * (3 * (l_max + 1) + 8)) * elem;
        unsigned fit = budget / per_point;
        S = fit >= 1 ? pow2_floor(fit) : 1;
        if (S > 64) S = 64;
        const int forced = env_int("SPHX_TILE", 0);
        if (forced > 0 && forced <= 64) S = static_cast<unsigned>(forced);
        per_group = S;
    }
    g.tile = static_cast<int>(S);
    plan->points_per_group = per_group;

    // LDS carve-up (elements)
    unsigned at = S * (ny + g.pad);
    at = (at + 3u) & ~3u;
    g.off_dsph = at;
    if (mode >= 1) at += S * (3 * ny + g.pad);
    at = (at + 3u) & ~3u;
    g.off_ddsph = at;
    if (mode == 2) at += S * (9 * ny + g.pad);
    at = (at + 3u) & ~3u;
    if (!plan->closed_form) {
        const unsigned nq = static_cast<unsigned>(l_max + 1) * (l_max + 2) / 2;
        g.off_F = at;
        at += nq;
        g.off_Q = at;
        at += nq;
        g.off_pts = at; // per point: 8 coordinates-and-such, then c, s, 2(m+1)z; two buffers
        at += 2 * S * (3 * (l_max + 1) + 8);
        // segment length: the shortest that still gives every job its own lane (192 lanes run
        // the recursion jobs), so that the longest chain of dependent work is as short as possible
        const int hard = mode == 2 ? 1 : 6;
        static const unsigned candidates[] = {2, 3, 4, 6, 8, 12, 16, 24, 32, 65};
        unsigned chosen = 65, jobs = 0;
        const int forced_segment = env_int("SPHX_SEGMENT", 0);
        for (unsigned cand : candidates) {
            unsigned count = 0;
            for (int l = hard + 1; l <= l_max; ++l) count += static_cast<unsigned>(l) / cand + 1;
            if ((forced_segment > 1 && cand >= static_cast<unsigned>(forced_segment)) ||
                (forced_segment <= 1 && S * count <= 192) || cand == 65) {
                chosen = cand;
                jobs = count;
                break;
            }
        }
        g.segment = chosen;
        g.jobs_per_point = jobs;
        g.off_jobs = at;
        at += (jobs * 2 + static_cast<unsigned>(elem) - 1) / static_cast<unsigned>(elem);
    }
    plan->lds_bytes = at * static_cast<unsigned>(elem);
    if (plan->lds_bytes > static_cast<unsigned>(lds_limit)) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) + " with this many derivatives needs " +
                        std::to_string(plan->lds_bytes) + " bytes of LDS per point tile; the device offers " +
                        std::to_string(lds_limit));
    }

    const unsigned long long tiles = (n_samples + per_group - 1) / per_group;
    if (tiles > 0x7fffffffull) return fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    g.n_tiles = static_cast<unsigned>(tiles);
    for (int a = 0; a < 3; ++a) {
        const unsigned long long row = (a == 0 ? 1ull : (a == 1 ? 3ull : 9ull)) * ny;
        g.magic[a] = static_cast<unsigned>(((1ull << 32) + row - 1) / row); // unused when row == 1
    }

    if (plan->closed_form) {
        g.tiles_per_group = (g.n_tiles + 7u) / 8u;
        plan->workgroups = g.tiles_per_group * 8u;
    } else {
        unsigned per_cu = static_cast<unsigned>(lds_limit) / (plan->lds_bytes ? plan->lds_bytes : 1u);
        if (per_cu < 1) per_cu = 1;
        if (per_cu > 8) per_cu = 8; // 256 threads each: 2048 lanes per CU
        unsigned want = static_cast<unsigned>(cus) * per_cu;
        want = (want + 7u) & ~7u;
        unsigned need = (g.n_tiles + 7u) & ~7u;
        plan->workgroups = want < need ? want : need;
        if (plan->workgroups < 8) plan->workgroups = 8;
        g.tiles_per_group = (g.n_tiles + 7u) / 8u;
    }
    return SPHX_OK;
}

template <typename T, int MODE, bool NORM, int H>
static hipError_t launch_closed(const Plan& plan, const T* xyz, T* sph, T* dsph, T* ddsph,
                                hipStream_t stream) {
    auto kernel = closed_form_kernel<T, MODE, NORM, H>;
    if (plan.lds_bytes > 64u * 1024u) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(plan.lds_bytes));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3(plan.workgroups), dim3(plan.threads), plan.lds_bytes, stream,
                       plan.g, xyz, sph, dsph, ddsph);
    return hipGetLastError();
}

template <typename T, int MODE, bool NORM, int H>
static hipError_t launch_recursion(const Plan& plan, const T* xyz, T* sph, T* dsph, T* ddsph,
                                   hipStream_t stream) {
    auto kernel = recursion_kernel<T, MODE, NORM, H>;
    if (plan.lds_bytes > 64u * 1024u) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(plan.lds_bytes));
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(kernel, dim3(plan.workgroups), dim3(plan.threads), plan.lds_bytes, stream,
                       plan.g, xyz, sph, dsph, ddsph);
    return hipGetLastError();
}

template <typename T, int MODE, bool NORM>
static hipError_t dispatch(const Plan& plan, const T* xyz, T* sph, T* dsph, T* ddsph,
                           hipStream_t stream) {
    if (!plan.closed_form) {
        return launch_recursion<T, MODE, NORM, (MODE == 2 ? 1 : 6)>(plan, xyz, sph, dsph, ddsph, stream);
    }
    switch (plan.g.l_max) {
    case 0:
        return launch_closed<T, MODE, NORM, 0>(plan, xyz, sph, dsph, ddsph, stream);
    case 1:
        return launch_closed<T, MODE, NORM, 1>(plan, xyz, sph, dsph, ddsph, stream);
    default:
        break;
    }
    if constexpr (MODE < 2) {
        switch (plan.g.l_max) {
        case 2:
            return launch_closed<T, MODE, NORM, 2>(plan, xyz, sph, dsph, ddsph, stream);
        case 3:
            return launch_closed<T, MODE, NORM, 3>(plan, xyz, sph, dsph, ddsph, stream);
        case 4:
            return launch_closed<T, MODE, NORM, 4>(plan, xyz, sph, dsph, ddsph, stream);
        case 5:
            return launch_closed<T, MODE, NORM, 5>(plan, xyz, sph, dsph, ddsph, stream);
        case 6:
            return launch_closed<T, MODE, NORM, 6>(plan, xyz, sph, dsph, ddsph, stream);
        default:
            break;
        }
    }
    return hipErrorInvalidValue;
}

template <typename T>
static int forward(const T* xyz, size_t n_samples, int l_max, int normalized, int mode, T* sph,
                   T* dsph, T* ddsph, void* stream) {
    t_error.clear();
    if (n_samples == 0) {
        return SPHX_OK;
    }
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (xyz == nullptr) return fail(SPHX_ERR_ARGUMENT, "xyz is a null pointer");
    if (sph == nullptr) return fail(SPHX_ERR_ARGUMENT, "sph is a null pointer");
    if (mode >= 1 && dsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "dsph is a null pointer");
    if (mode >= 2 && ddsph == nullptr) return fail(SPHX_ERR_ARGUMENT, "ddsph is a null pointer");

    hipPointerAttribute_t attr;
    SPHX_HIP(hipPointerGetAttributes(&attr, xyz));
    int current = 0;
    SPHX_HIP(hipGetDevice(&current));
    const int device = attr.device;
    if (device != current) {
        SPHX_HIP(hipSetDevice(device));
    }

    int status = ensure_device_ready(device);
    Plan plan;
    if (status == SPHX_OK) {
        status = make_plan(n_samples, l_max, mode, sizeof(T), g_lds_limit[device],
                           g_compute_units[device], &plan);
    }
    if (status == SPHX_OK) {
        hipStream_t s = reinterpret_cast<hipStream_t>(stream);
        hipError_t e;
        if (normalized) {
            e = mode == 0   ? dispatch<T, 0, true>(plan, xyz, sph, dsph, ddsph, s)
                : mode == 1 ? dispatch<T, 1, true>(plan, xyz, sph, dsph, ddsph, s)
                            : dispatch<T, 2, true>(plan, xyz, sph, dsph, ddsph, s);
        } else {
            e = mode == 0   ? dispatch<T, 0, false>(plan, xyz, sph, dsph, ddsph, s)
                : mode == 1 ? dispatch<T, 1, false>(plan, xyz, sph, dsph, ddsph, s)
                            : dispatch<T, 2, false>(plan, xyz, sph, dsph, ddsph, s);
        }
        if (e != hipSuccess) {
            status = fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
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

} // namespace sphx

extern "C" {

int sphx_forward_f32(const float* xyz, size_t n_samples, int l_max, int normalized,
                     int derivatives, float* sph, float* dsph, float* ddsph, void* stream) {
    return sphx::forward<float>(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph,
                                stream);
}

int sphx_forward_f64(const double* xyz, size_t n_samples, int l_max, int normalized,
                     int derivatives, double* sph, double* dsph, double* ddsph, void* stream) {
    return sphx::forward<double>(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph,
                                 stream);
}

int sphx_device_count(void) {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        sphx::t_error = std::string("hipGetDeviceCount: ") + hipGetErrorString(e);
        return -1;
    }
    return n;
}

const char* sphx_last_error(void) { return sphx::t_error.c_str(); }

int sphx_plan(size_t n_samples, int l_max, int derivatives, int is_f64, int* tile_samples,
              int* threads, int* lds_bytes, int* workgroups) {
    sphx::t_error.clear();
    int device = 0, lds = 160 * 1024, cus = 256;
    if (hipGetDevice(&device) == hipSuccess) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, device) == hipSuccess && v > 0) lds = v;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && v > 0) cus = v;
    } else {
        (void)hipGetLastError();
    }
    sphx::Plan plan;
    int status = sphx::make_plan(n_samples ? n_samples : 1, l_max, derivatives,
                                 is_f64 ? sizeof(double) : sizeof(float), lds, cus, &plan);
    if (status != SPHX_OK) return status;
    if (tile_samples) *tile_samples = static_cast<int>(plan.points_per_group);
    if (threads) *threads = plan.threads;
    if (lds_bytes) *lds_bytes = static_cast<int>(plan.lds_bytes);
    if (workgroups) *workgroups = static_cast<int>(plan.workgroups);
    return SPHX_OK;
}

} // extern "C"
