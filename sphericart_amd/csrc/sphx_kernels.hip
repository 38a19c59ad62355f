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
#include <type_traits>
#include <vector>

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
    unsigned n_tiles;       // tiles of `tile` points (recursion) or groups of 64 points (closed form)
    unsigned tiles_per_xcd; // workgroups of one XCD walk one contiguous stretch of tiles
    int l_max;
    int ny;                 // (l_max + 1)^2: length of one component row in HBM
    int tile;               // points whose rows are staged in LDS at a time
    unsigned magic_jobs;    // ceil(2^32 / jobs_per_point)
    unsigned jobs_per_point; // entry jobs per point: (l, m >= 0) pairs above the closed-form
                             // limit, or (l, m, side) triples when the sides are split
    unsigned sequence_waves; // waves that run the bare recursions (1 or 2)
    unsigned points_per_pass; // points whose entry jobs fit side by side in the wide waves (>= 1)
    unsigned vjp_accumulate; // fused product: add to xyz_grad instead of overwriting it
    unsigned az_shift;      // the point tables are made for 2^az_shift tiles at a time
    unsigned chunk_shift;   // a workgroup takes 2^chunk_shift consecutive tiles at a time
    unsigned row_buffers;   // 2: tile n is flushed while tile n+1 is computed; 1: one after the other
    unsigned flush_waves;   // waves that do nothing but flush (row_buffers == 2)
    // LDS carve-up, in elements of T: the row buffers come first, rows_elems each, with the
    // gradient and second-derivative rows at off_dsph and off_ddsph inside a buffer; the other
    // offsets count from the start of dynamic LDS
    unsigned rows_elems, off_dsph, off_ddsph, off_F, off_Q, off_pts, off_iter, off_jobs;
};

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

__host__ __device__ constexpr unsigned magic_of(unsigned long long divisor) {
    return static_cast<unsigned>(((1ull << 32) + divisor - 1) / divisor);
}

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
// Bytes of LDS one pass may use: 52 KB lets three workgroups share a CU. Measured on MI355X,
// l_max = 6 float32 with gradients runs fastest with a single pass (50 KB).
#ifndef SPHX_PHASE_LDS_BUDGET
#define SPHX_PHASE_LDS_BUDGET (52 * 1024)
#endif

__host__ __device__ constexpr unsigned components_of(int mode) {
    return mode == 0 ? 1u : (mode == 1 ? 4u : 13u);
}

// LDS elements per point in the closed-form kernel: the rows of all arrays, each array padded
// by one element when (H+1)^2 is even so that the per-point stride is odd (lanes staging the
// same entry of different points then hit different banks).
__host__ __device__ constexpr unsigned closed_form_pad(int H) {
    return ((H + 1) * (H + 1)) % 2 == 0 ? 1u : 0u;
}

__host__ __device__ constexpr unsigned closed_form_phases(unsigned elem, int mode, int H) {
    const unsigned ny = (H + 1) * (H + 1);
    const unsigned per_point = (components_of(mode) * ny + (mode + 1) * closed_form_pad(H)) * elem;
    unsigned phases = 1;
    while (phases < 16 && (64 / phases) * per_point > SPHX_PHASE_LDS_BUDGET) {
        phases *= 2;
    }
    return phases;
}

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

// ---------------------------------------------------------------------------
// Values only, l_max > 6, rows short enough that those of 64 points fit in LDS:
// 64 points per workgroup, one point per lane, one to eight waves that share
// the l channels of the same 64 points.
//
// Without derivatives an entry is three multiplications, so what counts is what
// surrounds them. With one point per lane l and m are the same for the whole
// wave: the prefactors come from constant memory through the scalar unit, no
// job has to be decoded and no iterate passes through LDS, about 15
// instructions per (l, +-m) pair of entries in all, a tenth of what the
// recursion kernel spends on them. (With derivatives the entries themselves
// dominate and rows are four and thirteen times as long, so that far fewer
// than 64 points fit: gradients_lanes_kernel takes l_max up to about 16, the
// recursion kernel the rest.)
//
// The rows of 64 points take most of a CU's LDS from l_max of about 12 on, and
// one wave would leave three of the four SIMDs idle: the l channels are dealt
// to the waves of the workgroup (in snake order, long and short ones mixed),
// each wave evaluating its channels for all 64 points (l_max = 15 float32,
// 500k points: 245 us with one wave, 113 with four, 106 with six). When not
// even 64 rows fit, 32 points per workgroup and half the lanes idle.
//
// Same operations in the same order as the reference: c_m, s_m, 2(m+1)z as in
// templates.hpp:451-466, l <= 6 in closed form, then per l the recursion of
// templates_core.hpp:122-123,155,202-204,393 downward in m, every iterate
// multiplied by its prefactor and by c_m and s_m (:127-128,160-162,214-218,395).
//
// LDS: the rows of the tile in HBM layout, so that the waves stream them out
// with 16-byte stores, and per point its table of (c_m, s_m, 2(m+1)z). A row
// length that is a multiple of 8 words would put the same entry of all points
// on few banks: such rows are kept one 16-byte vector apart.
// g.rows_elems: row stride, g.off_pts: start of the tables, g.off_iter: table stride.
// ---------------------------------------------------------------------------
constexpr unsigned kValuesMaxThreads = 512;

template <typename T, bool NORM>
__global__ __launch_bounds__(kValuesMaxThreads) void values_kernel(Tiling g, const T* __restrict__ xyz,
                                                                  T* __restrict__ sph) {
    constexpr int H = 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const unsigned waves = blockDim.x >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile); // 64, or fewer when 64 rows do not fit
    const unsigned long long first = static_cast<unsigned long long>(group) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    T* row = lds + lane * g.rows_elems;
    T* tab = lds + g.off_pts + lane * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    if (lane < valid) {
        p = load_point<T, NORM>(xyz + (first + lane) * 3);
        if (wave == 0) {
            const T twoz = p.z + p.z;
            T cm = 1.0, sm = 0.0, tz = twoz;
            tab[0] = cm;
            tab[1] = sm;
            tab[2] = tz;
            for (int m = 1; m <= L; ++m) {
                const T cn = cm * p.x - sm * p.y;
                const T sn = cm * p.y + sm * p.x;
                tz = tz + twoz;
                cm = cn;
                sm = sn;
                tab[3 * m] = cm;
                tab[3 * m + 1] = sm;
                tab[3 * m + 2] = tz;
            }
        }
        if (wave == waves - 1) { // the last wave gets the fewest channels below
            T Y[NYH];
            low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
#pragma unroll
            for (unsigned k = 0; k < NYH; ++k) row[k] = Y[k];
        }
    }
    __syncthreads(); // the tables
    if (lane < valid) {
        const T rxy = p.x2 + p.y2;
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        // channel number i = L - l goes to wave i % waves in even rounds, backwards in odd ones
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            const T* pk = cF + tri;
            const T* qk = cQ + tri;
            T* mid = row + l * l + l;
            T v2 = qk[l];
            T v1 = -p.z * v2;
            {
                const T pq = v2 * pk[l];
                mid[l] = pq * tab[3 * l];
                mid[-l] = pq * tab[3 * l + 1];
            }
            {
                const T pq = v1 * pk[l - 1];
                mid[l - 1] = pq * tab[3 * (l - 1)];
                mid[-(l - 1)] = pq * tab[3 * (l - 1) + 1];
            }
            for (int m = l - 2; m >= 1; --m) {
                const T v0 = qk[m] * (tab[3 * m + 2] * v1 + rxy * v2);
                const T pq = v0 * pk[m];
                mid[m] = pq * tab[3 * m];
                mid[-m] = pq * tab[3 * m + 1];
                v2 = v1;
                v1 = v0;
            }
            const T v0 = qk[0] * (tab[2] * v1 + rxy * v2);
            mid[0] = v0 * pk[0];
        }
    }
    __syncthreads(); // the rows
    T* dst = sph + first * ny;
    const unsigned len = valid * ny;
    const unsigned threads = blockDim.x;
    if (g.rows_elems == ny) {
        copy_out<T, SPHX_STREAMING_STORES, false, 1>(lds, dst, len, ny, 0, 0, tid, threads);
    } else if ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
        // rows one vector apart (their length is a whole number of vectors)
        const unsigned per_row = ny / W;
        const unsigned magic = magic_of(per_row);
        const V* in = reinterpret_cast<const V*>(lds);
        V* out = reinterpret_cast<V*>(dst);
        const unsigned nvec = len / W;
        for (unsigned v = tid; v < nvec; v += threads) {
            emit<T, SPHX_STREAMING_STORES>(in[v + __umulhi(v, magic)], out + v);
        }
    } else {
        for (unsigned e = tid; e < len; e += threads) {
            const unsigned r = e / ny;
            dst[e] = lds[e + r * (g.rows_elems - ny)];
        }
    }
}

// ---------------------------------------------------------------------------
// Values and gradients, l_max just above 6, where the four rows of 32 or 64 points
// still fit in LDS: the construction of values_kernel with the gradient entries
// added. One point per lane; wave 0 makes the (c_m, s_m, 2(m+1)z) tables; the
// closed forms of l <= 6 go in slices to the waves from the last one backwards,
// the l channels above to the waves in snake order; a lane runs the recursions
// of Q_l^m and Q_{l-1}^m in registers and stages the entries (l, +-m) of its point
// with the same functions as the recursion kernel (Entry, finish, put): same
// operations, same order, same numbers. All waves then stream out the two runs.
// g.rows_elems / g.off_dsph / g.off_ddsph: stride of a point's values row, start of
// the gradient rows, stride of a point's three gradient rows; g.off_pts, g.off_iter:
// the tables and their stride.
// ---------------------------------------------------------------------------
template <typename T, bool NORM>
__global__ __launch_bounds__(kValuesMaxThreads) void gradients_lanes_kernel(Tiling g, const T* __restrict__ xyz,
                                                                           T* __restrict__ sph,
                                                                           T* __restrict__ dsph) {
    constexpr int H = 6;
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const unsigned threads = blockDim.x;
    const unsigned waves = threads >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile);
    const unsigned long long first = static_cast<unsigned long long>(group) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    Rows<T> rows;
    rows.ny = static_cast<int>(ny);
    rows.sph = lds + lane * g.rows_elems;
    rows.dsph = lds + g.off_dsph + lane * g.off_ddsph;
    rows.ddsph = nullptr;
    T* tab = lds + g.off_pts + lane * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    if (lane < valid) {
        p = load_point<T, NORM>(xyz + (first + lane) * 3);
        if (wave == 0) {
            const T twoz = p.z + p.z;
            T cm = 1.0, sm = 0.0, tz = twoz;
            tab[0] = cm;
            tab[1] = sm;
            tab[2] = tz;
            for (int m = 1; m <= L; ++m) {
                const T cn = cm * p.x - sm * p.y;
                const T sn = cm * p.y + sm * p.x;
                tz = tz + twoz;
                cm = cn;
                sm = sn;
                tab[3 * m] = cm;
                tab[3 * m + 1] = sm;
                tab[3 * m + 2] = tz;
            }
        }
        const unsigned from_last = waves - 1u - wave;
        if (0 % waves == from_last) closed_form_job<T, 1, NORM, H, 0, 9>(p, rows);
        if (1 % waves == from_last) closed_form_job<T, 1, NORM, H, 9, 16>(p, rows);
        if (2 % waves == from_last) closed_form_job<T, 1, NORM, H, 16, 25>(p, rows);
        if (3 % waves == from_last) closed_form_job<T, 1, NORM, H, 25, 31>(p, rows);
        if (4 % waves == from_last) closed_form_job<T, 1, NORM, H, 31, 36>(p, rows);
        if (5 % waves == from_last) closed_form_job<T, 1, NORM, H, 36, 41>(p, rows);
        if (6 % waves == from_last) closed_form_job<T, 1, NORM, H, 41, 45>(p, rows);
        if (7 % waves == from_last) closed_form_job<T, 1, NORM, H, 45, 49>(p, rows);
    }
    __syncthreads(); // the tables
    if (lane < valid) {
        const T x = p.x, y = p.y;
        const T rxy = p.x2 + p.y2;
        const T zero = static_cast<T>(0.0);
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        auto entry = [&](T v, T gx, T gy, T gz) {
            Entry<T> e;
            e.v = v;
            e.gx = gx;
            e.gy = gy;
            e.gz = gz;
            e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = zero;
            return e;
        };
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            const int mid = 2 * tri;
            const T* pk = cF + tri;
            const T* qk = cQ + tri;
            const T* kb = qk - l; // constants of the Q_{l-1} recursion
            T a2 = qk[l];         // Q_l^l
            T a1 = -p.z * a2;     // Q_l^{l-1}
            T b2 = 0;             // the Q_{l-1} sequence: 0 at m = l,
            T b1 = qk[-1];        // Q_{l-1}^{l-1} at m = l - 1
            T c1 = tab[3 * (l - 1)], s1 = tab[3 * (l - 1) + 1];
            T c0 = tab[3 * l], s0 = tab[3 * l + 1];
            {
                // m = l (templates_core.hpp:122-152)
                auto pq = a2 * pk[l];
                const T vp = pq * c0, vn = pq * s0;
                pq *= l;
                stage<T, 1, NORM>(rows, mid + l, p, entry(vp, pq * c1, pq * -s1, zero));
                stage<T, 1, NORM>(rows, mid - l, p, entry(vn, pq * s1, pq * c1, zero));
            }
            c0 = c1;
            s0 = s1;
            c1 = tab[3 * (l - 2)];
            s1 = tab[3 * (l - 2) + 1];
            {
                // m = l - 1 (:154-198)
                const T pkm = pk[l - 1];
                auto pq = a1 * pkm;
                const T vp = pq * c0, vn = pq * s0;
                pq *= (l - 1);
                auto pdq = pkm * (l + l - 1) * b1;
                stage<T, 1, NORM>(rows, mid + l - 1, p, entry(vp, pq * c1, pq * -s1, pdq * c0));
                stage<T, 1, NORM>(rows, mid - (l - 1), p, entry(vn, pq * s1, pq * c1, pdq * s0));
            }
            for (int m = l - 2; m >= 1; --m) {
                // :201-390
                c0 = c1;
                s0 = s1;
                c1 = tab[3 * (m - 1)];
                s1 = tab[3 * (m - 1) + 1];
                const T tz = tab[3 * m + 2];
                const T a0 = qk[m] * (tz * a1 + rxy * a2);
                const T b0 = kb[m] * (tz * b1 + rxy * b2);
                const T pkm = pk[m];
                auto pq = a0 * pkm;
                const T vp = pq * c0, vn = pq * s0;
                pq *= m;
                auto pdq = pkm * b1;
                auto pdqx = pdq * x;
                auto pdqy = pdq * y;
                auto pdz = pkm * (l + m) * b0;
                stage<T, 1, NORM>(rows, mid + m, p,
                                  entry(vp, (pdqx * c0 + pq * c1), (pdqy * c0 + pq * -s1), pdz * c0));
                stage<T, 1, NORM>(rows, mid - m, p,
                                  entry(vn, (pdqx * s0 + pq * s1), (pdqy * s0 + pq * c1), pdz * s0));
                a2 = a1;
                a1 = a0;
                b2 = b1;
                b1 = b0;
            }
            {
                // m = 0 (:392-426)
                const T tz = tab[2];
                const T a0 = qk[0] * (tz * a1 + rxy * a2);
                const T b0 = kb[0] * (tz * b1 + rxy * b2);
                stage<T, 1, NORM>(rows, mid, p,
                                  entry(a0 * pk[0], pk[0] * x * b1, pk[0] * y * b1, pk[0] * l * b0));
            }
        }
    }
    __syncthreads(); // the rows
    // one run of valid * row elements per array; the points' blocks `stride` apart in LDS
    auto flush = [&](const T* staged, unsigned stride, unsigned row, T* dst) {
        const unsigned len = valid * row;
        if (stride == row) {
            copy_out<T, SPHX_STREAMING_STORES, false, 1>(staged, dst, len, row, 0, 0, tid, threads);
        } else if ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
            const unsigned per_row = row / W;
            const unsigned magic = magic_of(per_row);
            const V* in = reinterpret_cast<const V*>(staged);
            V* out = reinterpret_cast<V*>(dst);
            const unsigned nvec = len / W;
            for (unsigned v = tid; v < nvec; v += threads) {
                emit<T, SPHX_STREAMING_STORES>(in[v + __umulhi(v, magic)], out + v);
            }
        } else {
            for (unsigned e = tid; e < len; e += threads) dst[e] = staged[e + (e / row) * (stride - row)];
        }
    };
    flush(lds, g.rows_elems, ny, sph + first * ny);
    flush(lds + g.off_dsph, g.off_ddsph, 3 * ny, dsph + first * 3 * ny);
}

// ---------------------------------------------------------------------------
// Values, gradients and second derivatives for small l_max, where the thirteen
// rows of 32 or 64 points fit in LDS: one point per lane again, built from the
// recursion kernel's own jobs. A lane of wave 0 makes its point's c_m, s_m,
// 2(m+1)z (azimuth_job) while the last wave stages l <= 1 in closed form. The l
// channels are dealt to the waves in snake order; for a channel a lane runs the
// three bare recursions into a scratch of its own in LDS (sequence_job) and
// then turns every m into entries (entry_job), with no barrier in between. l
// and m are the same for all lanes of a wave, so the branches of entry_job are
// uniform and the prefactors come through the scalar unit; staging is free of
// bank conflicts as every lane writes the same entry of its own point. The
// arithmetic is the recursion kernel's, hence the reference's.
// g.rows_elems, g.off_dsph, g.off_ddsph strides, g.off_F, g.off_Q starts of the gradient and
// second-derivative rows; g.off_pts, g.off_iter: tables [c | s | 2(m+1)z] and their stride;
// g.off_jobs, g.jobs_per_point: the waves' scratch [A | B | C] and a lane's share of it.
// ---------------------------------------------------------------------------
constexpr unsigned kHessianLaneThreads = 256; // float64 entries need more than 128 registers

template <typename T, bool NORM>
__global__ __launch_bounds__(kHessianLaneThreads) void hessians_lanes_kernel(Tiling g, const T* __restrict__ xyz,
                                                                            T* __restrict__ sph,
                                                                            T* __restrict__ dsph,
                                                                            T* __restrict__ ddsph) {
    constexpr int H = 1;
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const unsigned threads = blockDim.x;
    const unsigned waves = threads >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile);
    const unsigned long long first = static_cast<unsigned long long>(group) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    Rows<T> rows;
    rows.ny = static_cast<int>(ny);
    rows.sph = lds + lane * g.rows_elems;
    rows.dsph = lds + g.off_F + lane * g.off_dsph;
    rows.ddsph = lds + g.off_Q + lane * g.off_ddsph;
    T* c = lds + g.off_pts + lane * g.off_iter;
    T* sn = c + (L + 1);
    T* tmz = sn + (L + 1);
    if (lane < valid) {
        p = load_point<T, NORM>(xyz + (first + lane) * 3);
        if (wave == 0) azimuth_job<T>(p, L, c, sn, tmz);
        if (wave == waves - 1) closed_form_job<T, 2, NORM, H>(p, rows);
    }
    __syncthreads(); // the tables
    if (lane < valid) {
        const T rxy = p.x2 + p.y2;
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        T* A = lds + g.off_jobs + (wave * tile + lane) * g.jobs_per_point;
        T* B = A + (L + 1);
        T* C = B + (L + 1);
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            sequence_job<T>(l, 0, p.z, rxy, cQ, tmz, A);
            sequence_job<T>(l, 1, p.z, rxy, cQ, tmz, B);
            sequence_job<T>(l, 2, p.z, rxy, cQ, tmz, C);
            for (int m = l; m >= 0; --m) {
                entry_job<T, 2, NORM, false>(l, m, tri, 0, p, cF + tri, c, sn, A, B, C, rows);
            }
        }
    }
    __syncthreads(); // the rows
    auto flush = [&](const T* staged, unsigned stride, unsigned row, T* dst) {
        const unsigned len = valid * row;
        if (stride == row) {
            copy_out<T, SPHX_STREAMING_STORES, false, 1>(staged, dst, len, row, 0, 0, tid, threads);
        } else if ((reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
            const unsigned per_row = row / W;
            const unsigned magic = magic_of(per_row);
            const V* in = reinterpret_cast<const V*>(staged);
            V* out = reinterpret_cast<V*>(dst);
            const unsigned nvec = len / W;
            for (unsigned v = tid; v < nvec; v += threads) {
                emit<T, SPHX_STREAMING_STORES>(in[v + __umulhi(v, magic)], out + v);
            }
        } else {
            for (unsigned e = tid; e < len; e += threads) dst[e] = staged[e + (e / row) * (stride - row)];
        }
    };
    flush(lds, g.rows_elems, ny, sph + first * ny);
    flush(lds + g.off_F, g.off_dsph, 3 * ny, dsph + first * 3 * ny);
    flush(lds + g.off_Q, g.off_ddsph, 9 * ny, ddsph + first * 9 * ny);
}

// ---------------------------------------------------------------------------
// Vector-Jacobian product without the Jacobian in memory, l_max <= 6:
//
//   xyz_grad[i][a] (+)= sum_k d sph[i][k] / d xyz[i][a] * sph_grad[i][k]
//
// Same evaluation as closed_form_kernel with gradients (one point per lane, the
// finished entries in VGPRs), but instead of staging 4 (l_max+1)^2 numbers per
// point for HBM the lane multiplies its gradient entries with the point's row of
// sph_grad and keeps three sums: (l_max+1)^2 + 3 numbers read and 3 written per
// point instead of 4 (l_max+1)^2 written and read again. LDS only turns the
// coalesced load of the tile's sph_grad rows into one row per lane (row stride
// odd, so the lanes hit different banks). The sums run over k in index order
// with one rounding per operation: the result is what contracting the
// gradients of the forward pass in that order gives, bit for bit.
// ---------------------------------------------------------------------------
//
// g.ny is the length of a row of sph_grad: (H+1)^2 when l_max = H; longer when this kernel
// takes only the first (H+1)^2 entries of every row and the recursion kernel adds the rest
// (recursion_kernel with VJP).
template <typename T, bool NORM, int H>
__global__ __launch_bounds__(64, 3) void closed_form_vjp_kernel(Tiling g, const T* __restrict__ xyz,
                                                            const T* __restrict__ sph_grad,
                                                            T* __restrict__ xyz_grad, int accumulate) {
    constexpr unsigned NY = (H + 1) * (H + 1);
    constexpr unsigned STRIDE = NY + closed_form_pad(H);
    T* weights = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned long long first = static_cast<unsigned long long>(group) * 64;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < 64ull ? static_cast<unsigned>(left) : 64u;

    // l_max = H: the tile's rows of sph_grad are one contiguous run: consecutive lanes,
    // consecutive addresses
    const unsigned row_stride = static_cast<unsigned>(g.ny);
    const T* run = sph_grad + first * row_stride;
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    const unsigned total = valid * NY;
    if (row_stride != NY) {
        for (unsigned i = tid; i < total; i += 64) {
            const unsigned s = i / NY;
            weights[i + (STRIDE - NY) * s] = run[static_cast<unsigned long long>(s) * row_stride + (i - s * NY)];
        }
    } else if ((reinterpret_cast<uintptr_t>(run) & 15u) == 0 && total % W == 0) {
        const V* in = reinterpret_cast<const V*>(run);
        for (unsigned v = tid; v < total / W; v += 64) {
            const V four = in[v];
#pragma unroll
            for (unsigned e = 0; e < W; ++e) {
                const unsigned i = v * W + e;
                weights[i + (STRIDE - NY) * (i / NY)] = four[e];
            }
        }
    } else {
        for (unsigned i = tid; i < total; i += 64) {
            weights[i + (STRIDE - NY) * (i / NY)] = run[i];
        }
    }
    __syncthreads();
    if (tid >= valid) return;

    const Point<T> p = load_point<T, NORM>(xyz + (first + tid) * 3);
    const T* mine = weights + tid * STRIDE;
    T sum_x = 0, sum_y = 0, sum_z = 0;
    // The entries in slices, one after the other in index order: a slice evaluates little more
    // than its own entries (see closed_form_job), so that far fewer numbers are alive at a time
    // than with all 3 x 49 gradient entries of a point in registers (float64: 340 registers and
    // one wave per SIMD before). Same entries, same order of the additions.
    auto slice = [&](auto lo, auto hi) {
        constexpr int KLO = decltype(lo)::value, KHI = decltype(hi)::value;
        T Y[NY], DX[NY], DY[NY], DZ[NY];
        low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
        low_gradients<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y, DX, DY, DZ);
#pragma unroll
        for (int k = KLO; k < KHI; ++k) {
            Entry<T> e;
            e.v = Y[k];
            e.gx = DX[k];
            e.gy = DY[k];
            e.gz = DZ[k];
            e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = static_cast<T>(0.0);
            e = finish<T, 1, NORM>(p, e);
            const T wk = mine[k];
            sum_x += e.gx * wk;
            sum_y += e.gy * wk;
            sum_z += e.gz * wk;
        }
    };
    using std::integral_constant;
    if constexpr (H == 6) {
        slice(integral_constant<int, 0>{}, integral_constant<int, 16>{});
        slice(integral_constant<int, 16>{}, integral_constant<int, 25>{});
        slice(integral_constant<int, 25>{}, integral_constant<int, 36>{});
        slice(integral_constant<int, 36>{}, integral_constant<int, 42>{});
        slice(integral_constant<int, 42>{}, integral_constant<int, 49>{});
    } else {
        slice(integral_constant<int, 0>{}, integral_constant<int, static_cast<int>(NY)>{});
    }
    T* out = xyz_grad + (first + tid) * 3;
    if (accumulate) {
        sum_x += out[0];
        sum_y += out[1];
        sum_z += out[2];
    }
    out[0] = sum_x;
    out[1] = sum_y;
    out[2] = sum_z;
}

// ---------------------------------------------------------------------------
// Vector-Jacobian product, l_max > 6, one point per lane (the construction of
// values_kernel): what passes through LDS is the tile's rows of sph_grad, read
// from HBM with consecutive lanes at consecutive addresses, and the per-point
// tables; the gradient entries never leave the registers. A lane runs the two
// recursions a gradient needs (Q_l^m and Q_{l-1}^m, templates_core.hpp:202-212),
// forms the entries (l, +-m) of the three gradient rows as the reference does
// (:129-133, :163-170, :219-227, :396-399), multiplies them with the two
// weights and adds to three sums. The chain rule of the normalised harmonics is
// linear in the gradient (templates.hpp:608-612), so it is applied once, to the
// sums. The l channels are dealt to the waves as in values_kernel; the last
// wave also takes l <= 6 in closed form; the waves' sums meet in LDS and wave 0
// adds them in a fixed order. The terms are added in another order than a
// sequential loop over k would, so the result agrees with the contraction of
// the forward gradients to rounding, not bit for bit.
// g.rows_elems: row stride of the staged weights, g.off_pts: tables,
// g.off_iter: table stride, g.off_jobs: the waves' sums.
// ---------------------------------------------------------------------------
template <typename T, bool NORM>
__global__ __launch_bounds__(kValuesMaxThreads) void vjp_lanes_kernel(Tiling g, const T* __restrict__ xyz,
                                                                     const T* __restrict__ sph_grad,
                                                                     T* __restrict__ xyz_grad,
                                                                     int accumulate) {
    constexpr int H = 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const unsigned threads = blockDim.x;
    const unsigned waves = threads >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile);
    const unsigned long long first = static_cast<unsigned long long>(group) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    // the tile's rows of sph_grad, one contiguous run, into LDS (rows `rows_elems` apart)
    {
        const T* run = sph_grad + first * ny;
        const unsigned len = valid * ny;
        const unsigned gap = g.rows_elems - ny;
        if ((reinterpret_cast<uintptr_t>(run) & 15u) == 0 && (gap == 0 || ny % W == 0)) {
            const V* in = reinterpret_cast<const V*>(run);
            V* staged = reinterpret_cast<V*>(lds);
            const unsigned nvec = len / W;
            const unsigned magic = magic_of(ny / W ? ny / W : 1u);
            // many loads in flight per lane: the tile is read once, and with one load at a
            // time the latency of HBM, several times over, was most of a large tile's time
            constexpr unsigned DEPTH = 8;
            unsigned v = tid;
            for (; v + (DEPTH - 1) * threads < nvec; v += DEPTH * threads) {
                V hold[DEPTH];
#pragma unroll
                for (unsigned u = 0; u < DEPTH; ++u) hold[u] = in[v + u * threads];
#pragma unroll
                for (unsigned u = 0; u < DEPTH; ++u) {
                    const unsigned at = v + u * threads;
                    staged[gap == 0 ? at : at + __umulhi(at, magic) * (gap / W)] = hold[u];
                }
            }
            for (; v < nvec; v += threads) {
                staged[gap == 0 ? v : v + __umulhi(v, magic) * (gap / W)] = in[v];
            }
            for (unsigned e = nvec * W + tid; e < len; e += threads) lds[e] = run[e]; // gap == 0 only
        } else {
            for (unsigned e = tid; e < len; e += threads) {
                lds[e + (e / ny) * gap] = run[e];
            }
        }
    }

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    const T* weight = lds + lane * g.rows_elems;
    T* tab = lds + g.off_pts + lane * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    if (lane < valid) {
        p = load_point<T, NORM>(xyz + (first + lane) * 3);
        if (wave == 0) {
            const T twoz = p.z + p.z;
            T cm = 1.0, sm = 0.0, tz = twoz;
            tab[0] = cm;
            tab[1] = sm;
            tab[2] = tz;
            for (int m = 1; m <= L; ++m) {
                const T cn = cm * p.x - sm * p.y;
                const T sn = cm * p.y + sm * p.x;
                tz = tz + twoz;
                cm = cn;
                sm = sn;
                tab[3 * m] = cm;
                tab[3 * m + 1] = sm;
                tab[3 * m + 2] = tz;
            }
        }
    }
    __syncthreads(); // weights and tables

    T sum_x = 0, sum_y = 0, sum_z = 0;
    if (lane < valid) {
        const T x = p.x, y = p.y;
        const T rxy = p.x2 + p.y2;
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            const T* pk = cF + tri;
            const T* qk = cQ + tri;
            const T* kb = qk - l; // constants of the Q_{l-1} recursion
            const T* wmid = weight + l * l + l;
            // the entries (l, +m) and (l, -m) of the gradient rows times their weights
            auto add = [&](int m, T gx_pos, T gy_pos, T gz_pos, T gx_neg, T gy_neg, T gz_neg) {
                const T wp = wmid[m], wn = wmid[-m];
                sum_x += gx_pos * wp;
                sum_y += gy_pos * wp;
                sum_z += gz_pos * wp;
                sum_x += gx_neg * wn;
                sum_y += gy_neg * wn;
                sum_z += gz_neg * wn;
            };
            T a2 = qk[l];       // Q_l^l
            T a1 = -p.z * a2;   // Q_l^{l-1}
            T b2 = 0;           // the Q_{l-1} sequence: 0 at m = l,
            T b1 = qk[-1];      // Q_{l-1}^{l-1} at m = l - 1
            T c1 = tab[3 * (l - 1)], s1 = tab[3 * (l - 1) + 1]; // c, s at m - 1 of the step at hand
            {
                // m = l
                T pq = a2 * pk[l];
                pq *= l;
                add(l, pq * c1, pq * -s1, T(0), pq * s1, pq * c1, T(0));
            }
            T c0 = c1, s0 = s1; // c, s at m
            c1 = tab[3 * (l - 2)];
            s1 = tab[3 * (l - 2) + 1];
            {
                // m = l - 1
                const T pkm = pk[l - 1];
                T pq = a1 * pkm;
                pq *= (l - 1);
                const T pdq = pkm * (l + l - 1) * b1;
                add(l - 1, pq * c1, pq * -s1, pdq * c0, pq * s1, pq * c1, pdq * s0);
            }
            for (int m = l - 2; m >= 1; --m) {
                c0 = c1;
                s0 = s1;
                c1 = tab[3 * (m - 1)];
                s1 = tab[3 * (m - 1) + 1];
                const T tz = tab[3 * m + 2];
                const T a0 = qk[m] * (tz * a1 + rxy * a2);
                const T b0 = kb[m] * (tz * b1 + rxy * b2);
                const T pkm = pk[m];
                T pq = a0 * pkm;
                pq *= m;
                const T pdq = pkm * b1;
                const T pdqx = pdq * x;
                const T pdqy = pdq * y;
                const T pdz = pkm * (l + m) * b0;
                add(m, pdqx * c0 + pq * c1, pdqy * c0 + pq * -s1, pdz * c0,
                    pdqx * s0 + pq * s1, pdqy * s0 + pq * c1, pdz * s0);
                a2 = a1;
                a1 = a0;
                b2 = b1;
                b1 = b0;
            }
            {
                // m = 0
                const T b0 = kb[0] * (tab[2] * b1 + rxy * b2);
                const T w0 = wmid[0];
                sum_x += pk[0] * x * b1 * w0;
                sum_y += pk[0] * y * b1 * w0;
                sum_z += pk[0] * l * b0 * w0;
            }
        }
        // l <= 6 in closed form, in slices of entries that go to the waves from the last one
        // backwards (those have the fewest channels above); a slice evaluates little more than
        // its own entries, see closed_form_job
        auto closed_slice = [&](auto lo, auto hi) {
            constexpr int KLO = decltype(lo)::value, KHI = decltype(hi)::value;
            T Y[NYH], DX[NYH], DY[NYH], DZ[NYH];
            low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
            low_gradients<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y, DX, DY, DZ);
#pragma unroll
            for (int k = KLO; k < KHI; ++k) {
                const T wk = weight[k];
                sum_x += DX[k] * wk;
                sum_y += DY[k] * wk;
                sum_z += DZ[k] * wk;
            }
        };
        const unsigned from_last = waves - 1u - wave;
        using std::integral_constant;
        if (0 % waves == from_last) closed_slice(integral_constant<int, 0>{}, integral_constant<int, 9>{});
        if (1 % waves == from_last) closed_slice(integral_constant<int, 9>{}, integral_constant<int, 16>{});
        if (2 % waves == from_last) closed_slice(integral_constant<int, 16>{}, integral_constant<int, 25>{});
        if (3 % waves == from_last) closed_slice(integral_constant<int, 25>{}, integral_constant<int, 31>{});
        if (4 % waves == from_last) closed_slice(integral_constant<int, 31>{}, integral_constant<int, 36>{});
        if (5 % waves == from_last) closed_slice(integral_constant<int, 36>{}, integral_constant<int, 41>{});
        if (6 % waves == from_last) closed_slice(integral_constant<int, 41>{}, integral_constant<int, 45>{});
        if (7 % waves == from_last) closed_slice(integral_constant<int, 45>{}, integral_constant<int, 49>{});
    }
    // the waves' sums: [wave][component][point]
    T* partial = lds + g.off_jobs;
    if (wave != 0 && lane < valid) {
        partial[(wave * 3 + 0) * tile + lane] = sum_x;
        partial[(wave * 3 + 1) * tile + lane] = sum_y;
        partial[(wave * 3 + 2) * tile + lane] = sum_z;
    }
    __syncthreads();
    if (wave == 0 && lane < valid) {
        for (unsigned w = 1; w < waves; ++w) {
            sum_x += partial[(w * 3 + 0) * tile + lane];
            sum_y += partial[(w * 3 + 1) * tile + lane];
            sum_z += partial[(w * 3 + 2) * tile + lane];
        }
        if constexpr (NORM) {
            const T tmp = sum_x * p.x + sum_y * p.y + sum_z * p.z;
            sum_x = (sum_x - p.x * tmp) * p.ir;
            sum_y = (sum_y - p.y * tmp) * p.ir;
            sum_z = (sum_z - p.z * tmp) * p.ir;
        }
        T* out = xyz_grad + (first + lane) * 3;
        if (accumulate) {
            sum_x += out[0];
            sum_y += out[1];
            sum_z += out[2];
        }
        out[0] = sum_x;
        out[1] = sum_y;
        out[2] = sum_z;
    }
}

// ---------------------------------------------------------------------------
// vjp_lanes_kernel for tiles of fewer than 64 points (the rows of sph_grad of 64
// points no longer fit in LDS): a wave's lanes are 64 / tile groups of `tile`
// lanes, every group with the same points and an l channel of its own, so that
// no lane idles. l then differs within the wave: the prefactors come from
// copies of the tables in LDS (one address per group) instead of the scalar
// unit, and the groups of a wave, which take consecutive l, run one loop over m
// from the largest l down, each lane joining at its own m = l.
// g.off_F, g.off_Q: the tables; the waves' sums at g.off_jobs are
// [wave][group][component][point].
// ---------------------------------------------------------------------------
template <typename T, bool NORM>
__global__ __launch_bounds__(kValuesMaxThreads) void vjp_groups_kernel(Tiling g, const T* __restrict__ xyz,
                                                                      const T* __restrict__ sph_grad,
                                                                      T* __restrict__ xyz_grad,
                                                                      int accumulate) {
    constexpr int H = 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const unsigned threads = blockDim.x;
    const unsigned waves = threads >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group_of_tiles = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group_of_tiles >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile);
    const unsigned groups = 64u / tile;           // lane groups per wave
    const unsigned point = lane % tile;           // this lane's point within the tile
    const unsigned group = lane / tile;           // this lane's group within the wave
    const unsigned long long first = static_cast<unsigned long long>(group_of_tiles) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    {
        const T* run = sph_grad + first * ny;
        const unsigned len = valid * ny;
        const unsigned gap = g.rows_elems - ny;
        if ((reinterpret_cast<uintptr_t>(run) & 15u) == 0 && (gap == 0 || ny % W == 0)) {
            const V* in = reinterpret_cast<const V*>(run);
            V* staged = reinterpret_cast<V*>(lds);
            const unsigned nvec = len / W;
            const unsigned magic = magic_of(ny / W ? ny / W : 1u);
            // many loads in flight per lane: the tile is read once, and with one load at a
            // time the latency of HBM, several times over, was most of a large tile's time
            constexpr unsigned DEPTH = 8;
            unsigned v = tid;
            for (; v + (DEPTH - 1) * threads < nvec; v += DEPTH * threads) {
                V hold[DEPTH];
#pragma unroll
                for (unsigned u = 0; u < DEPTH; ++u) hold[u] = in[v + u * threads];
#pragma unroll
                for (unsigned u = 0; u < DEPTH; ++u) {
                    const unsigned at = v + u * threads;
                    staged[gap == 0 ? at : at + __umulhi(at, magic) * (gap / W)] = hold[u];
                }
            }
            for (; v < nvec; v += threads) {
                staged[gap == 0 ? v : v + __umulhi(v, magic) * (gap / W)] = in[v];
            }
            for (unsigned e = nvec * W + tid; e < len; e += threads) lds[e] = run[e];
        } else {
            for (unsigned e = tid; e < len; e += threads) {
                lds[e + (e / ny) * gap] = run[e];
            }
        }
        const unsigned tri_all = static_cast<unsigned>((L + 1) * (L + 2) / 2);
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        for (unsigned i = tid; i < tri_all; i += threads) {
            lds[g.off_F + i] = cF[i];
            lds[g.off_Q + i] = cQ[i];
        }
    }

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    const T* weight = lds + point * g.rows_elems;
    T* tab = lds + g.off_pts + point * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    const bool has_point = point < valid;
    if (has_point) {
        p = load_point<T, NORM>(xyz + (first + point) * 3);
        if (wave == 0 && group == 0) {
            const T twoz = p.z + p.z;
            T cm = 1.0, sm = 0.0, tz = twoz;
            tab[0] = cm;
            tab[1] = sm;
            tab[2] = tz;
            for (int m = 1; m <= L; ++m) {
                const T cn = cm * p.x - sm * p.y;
                const T sn = cm * p.y + sm * p.x;
                tz = tz + twoz;
                cm = cn;
                sm = sn;
                tab[3 * m] = cm;
                tab[3 * m + 1] = sm;
                tab[3 * m + 2] = tz;
            }
        }
    }
    __syncthreads(); // weights, tables

    T sum_x = 0, sum_y = 0, sum_z = 0;
    const T x = p.x, y = p.y;
    const T rxy = p.x2 + p.y2;
    const unsigned channels = static_cast<unsigned>(L - H);
    const unsigned slots = (channels + groups - 1u) / groups; // a slot: `groups` consecutive channels
    for (unsigned j = 0; j < slots; ++j) {
        const unsigned pos = j % waves;
        if ((((j / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue; // snake over the waves
        const unsigned i = j * groups + group;      // channel number: l = L - i
        const bool active = has_point && i < channels;
        const int l = L - static_cast<int>(i);
        const int l_top = L - static_cast<int>(j * groups); // the largest l of the slot
        const int tri = active ? l * (l + 1) / 2 : 0;
        const T* pk = lds + g.off_F + tri;
        const T* qk = lds + g.off_Q + tri;
        const T* kb = qk - l;
        const T* wmid = weight + (active ? l * l + l : 0);
        auto add = [&](int m, T gx_pos, T gy_pos, T gz_pos, T gx_neg, T gy_neg, T gz_neg) {
            const T wp = wmid[m], wn = wmid[-m];
            sum_x += gx_pos * wp;
            sum_y += gy_pos * wp;
            sum_z += gz_pos * wp;
            sum_x += gx_neg * wn;
            sum_y += gy_neg * wn;
            sum_z += gz_neg * wn;
        };
        T a2 = 0, a1 = 0, b2 = 0, b1 = 0; // Q_l and Q_{l-1} at m + 2, m + 1
        T c_hi = 0, s_hi = 0;             // c_m, s_m, carried from the step before
        auto general = [&](int m) {
            const T c_lo = tab[3 * (m - 1)], s_lo = tab[3 * (m - 1) + 1];
            const T tz = tab[3 * m + 2];
            const T a0 = qk[m] * (tz * a1 + rxy * a2);
            const T b0 = kb[m] * (tz * b1 + rxy * b2);
            const T pkm = pk[m];
            T pq = a0 * pkm;
            pq *= m;
            const T pdq = pkm * b1;
            const T pdqx = pdq * x;
            const T pdqy = pdq * y;
            const T pdz = pkm * (l + m) * b0;
            add(m, pdqx * c_hi + pq * c_lo, pdqy * c_hi + pq * -s_lo, pdz * c_hi,
                pdqx * s_hi + pq * s_lo, pdqy * s_hi + pq * c_lo, pdz * s_hi);
            a2 = a1;
            a1 = a0;
            b2 = b1;
            b1 = b0;
            c_hi = c_lo;
            s_hi = s_lo;
        };
        // the first steps, in which the groups join one after the other (m = l, then m = l - 1)
        int m = l_top;
        const int joined = l_top - static_cast<int>(groups); // from here down every lane is in the bulk
        for (; m >= joined && m >= 1; --m) {
            if (!active || m > l) continue;
            if (m == l) {
                const T c_lo = tab[3 * (m - 1)], s_lo = tab[3 * (m - 1) + 1];
                a2 = qk[l];
                a1 = -p.z * a2;
                b2 = 0;
                b1 = qk[-1];
                T pq = a2 * pk[l];
                pq *= l;
                add(l, pq * c_lo, pq * -s_lo, T(0), pq * s_lo, pq * c_lo, T(0));
                c_hi = c_lo;
                s_hi = s_lo;
            } else if (m == l - 1) {
                const T c_lo = tab[3 * (m - 1)], s_lo = tab[3 * (m - 1) + 1];
                const T pkm = pk[m];
                T pq = a1 * pkm;
                pq *= m;
                const T pdq = pkm * (l + l - 1) * b1;
                add(m, pq * c_lo, pq * -s_lo, pdq * c_hi, pq * s_lo, pq * c_lo, pdq * s_hi);
                c_hi = c_lo;
                s_hi = s_lo;
            } else {
                general(m);
            }
        }
        // the bulk: the same straight-line step for every lane
        if (active) {
#pragma unroll 2
            for (; m >= 1; --m) general(m);
        }
        if (active) {
            // m = 0
            const T b0 = kb[0] * (tab[2] * b1 + rxy * b2);
            const T w0 = wmid[0];
            sum_x += pk[0] * x * b1 * w0;
            sum_y += pk[0] * y * b1 * w0;
            sum_z += pk[0] * l * b0 * w0;
        }
    }
    if (has_point && group == 0) {
        // l <= 6 in closed form, slices dealt to the waves from the last one backwards
        auto closed_slice = [&](auto lo, auto hi) {
            constexpr int KLO = decltype(lo)::value, KHI = decltype(hi)::value;
            T Y[NYH], DX[NYH], DY[NYH], DZ[NYH];
            low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
            low_gradients<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y, DX, DY, DZ);
#pragma unroll
            for (int k = KLO; k < KHI; ++k) {
                const T wk = weight[k];
                sum_x += DX[k] * wk;
                sum_y += DY[k] * wk;
                sum_z += DZ[k] * wk;
            }
        };
        const unsigned from_last = waves - 1u - wave;
        using std::integral_constant;
        if (0 % waves == from_last) closed_slice(integral_constant<int, 0>{}, integral_constant<int, 9>{});
        if (1 % waves == from_last) closed_slice(integral_constant<int, 9>{}, integral_constant<int, 16>{});
        if (2 % waves == from_last) closed_slice(integral_constant<int, 16>{}, integral_constant<int, 25>{});
        if (3 % waves == from_last) closed_slice(integral_constant<int, 25>{}, integral_constant<int, 31>{});
        if (4 % waves == from_last) closed_slice(integral_constant<int, 31>{}, integral_constant<int, 36>{});
        if (5 % waves == from_last) closed_slice(integral_constant<int, 36>{}, integral_constant<int, 41>{});
        if (6 % waves == from_last) closed_slice(integral_constant<int, 41>{}, integral_constant<int, 45>{});
        if (7 % waves == from_last) closed_slice(integral_constant<int, 45>{}, integral_constant<int, 49>{});
    }
    // every lane's sums: [wave][component][lane]; lane `point` of wave 0 adds those of its point
    T* partial = lds + g.off_jobs;
    partial[(wave * 3 + 0) * 64 + lane] = sum_x;
    partial[(wave * 3 + 1) * 64 + lane] = sum_y;
    partial[(wave * 3 + 2) * 64 + lane] = sum_z;
    __syncthreads();
    if (wave == 0 && group == 0 && has_point) {
        T total_x = 0, total_y = 0, total_z = 0;
        for (unsigned w = 0; w < waves; ++w) {
            for (unsigned q = 0; q < groups; ++q) {
                total_x += partial[(w * 3 + 0) * 64 + q * tile + point];
                total_y += partial[(w * 3 + 1) * 64 + q * tile + point];
                total_z += partial[(w * 3 + 2) * 64 + q * tile + point];
            }
        }
        if constexpr (NORM) {
            const T tmp = total_x * p.x + total_y * p.y + total_z * p.z;
            total_x = (total_x - p.x * tmp) * p.ir;
            total_y = (total_y - p.y * tmp) * p.ir;
            total_z = (total_z - p.z * tmp) * p.ir;
        }
        T* out = xyz_grad + (first + point) * 3;
        if (accumulate) {
            total_x += out[0];
            total_y += out[1];
            total_z += out[2];
        }
        out[0] = total_x;
        out[1] = total_y;
        out[2] = total_z;
    }
}

// ---------------------------------------------------------------------------
// l > H through the recursion. 512 threads, persistent workgroups that walk
// over tiles of `tile` consecutive points, four tiles in flight per workgroup,
// every wave with a role of its own and one barrier per tile:
//
//   wave 0       one batch of up to eight tiles ahead, one lane per point:
//                normalised coordinates, c_m, s_m, 2(m+1)z into LDS (azimuth_job);
//   wave 1 (, 2) tile i+1, one lane per (point, l, sequence): the bare Q recursions,
//                every iterate into LDS (sequence_job);
//   entry waves  tile i, one job per (point, l, m >= 0): the entries (l, +-m) of
//                every requested array, chain rule included, staged in LDS in
//                HBM layout (entry_job). Neighbouring lanes take neighbouring m
//                of one (point, l), so their LDS traffic falls on neighbouring
//                banks;
//   flush waves  tile i-1: stream its staged rows to HBM with 16-byte stores.
//
// The first two stages are short chains of dependent operations that only a
// few lanes can share; running them one and two tiles ahead of the wide stage
// takes them off the critical path. The last stage is bound by HBM, the entry
// stage by the vector ALUs: side by side, neither waits for the other. The
// point tables are kept in three buffers, the iterates and the staged rows in
// two. When the rows of a single point are too long for two row buffers there
// is one, no wave is set aside for flushing, and all waves flush tile i after
// a second barrier.
//
// SPLIT == true (second derivatives, so few points per tile that the (l, m)
// pairs of a tile leave lanes idle): the entries (l, +m) and (l, -m) are two
// jobs.
//
// WHOLE == true: the closed forms of l <= H are evaluated here too (one lane
// per point, the entries in slices that go round all waves) and the tile's
// rows are complete, one contiguous run per array.
// WHOLE == false: the rows start at l = H + 1 (closed_form_kernel<PREFIX>
// writes the part below); every (point, component) row is its own run.
// ---------------------------------------------------------------------------
constexpr unsigned kRecursionThreads = 512;

// Values and gradients: at most 128 registers, so that two workgroups share a CU (four waves
// per SIMD) wherever their LDS allows. Only the float64 closed forms exceed that on their own
// and spill a few registers; with 170 registers and one workgroup per CU, l_max = 12 float64
// gradients took 800 us instead of 513 us. The second-derivative kernels keep what they need
// (forced to 128 they spill in the entry jobs: 918 us against 558 us at l_max = 10, float64).
template <typename T, int MODE, bool NORM, bool WHOLE, bool SPLIT, bool VJP = false>
__global__ __launch_bounds__(kRecursionThreads, MODE < 2 ? 4 : 1) void recursion_kernel(Tiling g, const T* __restrict__ xyz,
                                                                     T* __restrict__ sph,
                                                                     T* __restrict__ dsph,
                                                                     T* __restrict__ ddsph) {
    static_assert(!VJP || (MODE == 1 && !SPLIT), "the fused product is built on the gradient kernel");
    constexpr int H = MODE == 2 ? 1 : 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    constexpr unsigned ARRAYS = MODE + 1; // iterate arrays per point: A, B, C
    constexpr unsigned NT = kRecursionThreads;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = tid >> 6;
    const int L = g.l_max;
    const unsigned S = g.tile;
    const unsigned ny = g.ny;
    const unsigned nrow = WHOLE ? ny : ny - NYH; // staged elements per component row
    const unsigned skip = WHOLE ? 0u : NYH;      // first staged entry of a row
    // Distance between staged rows. WHOLE == false: the rows are ny apart in HBM but only nrow
    // long; a stride that equals ny modulo 16 bytes, with the first row placed like its HBM
    // address modulo 16 bytes, puts every staged row at the same position within 16 bytes as
    // its destination, so that the copy is 16-byte loads and stores on both sides.
    constexpr unsigned W16 = 16u / static_cast<unsigned>(sizeof(T));
    const unsigned row_stride = nrow + skip % W16;
    const unsigned tri_all = (L + 1) * (L + 2) / 2;

    T* F = lds + g.off_F;
    T* Q = lds + g.off_Q;
    unsigned* job_table = reinterpret_cast<unsigned*>(lds + g.off_jobs);
    {
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        for (unsigned i = tid; i < tri_all; i += NT) {
            F[i] = cF[i];
            Q[i] = cQ[i];
        }
        // (l, m) pairs: the bulk 1 <= m <= l - 2 first, then the special cases m = l, l - 1 and
        // 0 each as one block, so that the lanes of a wave mostly share one branch of entry_job
        // one word per job: m in bits 0-6, the side in bit 7, l in bits 8-15, l(l+1)/2 above
        auto pack = [](int l, int m, int side) -> unsigned {
            return (static_cast<unsigned>(l * (l + 1) / 2) << 16) | (static_cast<unsigned>(l) << 8) |
                   (static_cast<unsigned>(side) << 7) | static_cast<unsigned>(m);
        };
        // one thread per l fills that l's places (a single thread writing all of them took
        // 10 us at l_max = 32, a third of the time of a small evaluation)
        if (static_cast<int>(tid) < L - H) {
            constexpr unsigned SIDES = SPLIT ? 2u : 1u;
            const int l = L - static_cast<int>(tid);
            const unsigned levels = static_cast<unsigned>(L - H);
            auto bulk_above = [&](int from) { // sum of (l' - 2) over from < l' <= L
                return static_cast<unsigned>(L * (L + 1) / 2 - from * (from + 1) / 2 - 2 * (L - from));
            };
            const unsigned bulk_all = bulk_above(H);
            for (unsigned side = 0; side < SIDES; ++side) {
                unsigned at = side * bulk_all + bulk_above(l);
                for (int m = l - 2; m >= 1; --m) job_table[at++] = pack(l, m, static_cast<int>(side));
                job_table[SIDES * bulk_all + side * levels + tid] = pack(l, l, static_cast<int>(side));
                job_table[SIDES * (bulk_all + levels) + side * levels + tid] = pack(l, l - 1, static_cast<int>(side));
            }
            job_table[SIDES * (bulk_all + 2 * levels) + tid] = pack(l, 0, 0);
        }
    }

    // per point: 8 numbers (x, y, z, x^2, y^2, z^2, 1/r, x^2 + y^2), then c, s, 2(m+1)z
    const unsigned point_stride = 8 + 3 * (L + 1);
    // The tables are made for 2^az_shift tiles at a time (a batch), one lane per point, so that
    // the recurrences, a chain of dependent operations that few lanes share, run once per batch
    // instead of once per tile. Single tiles are made two rounds ahead and kept in three
    // buffers; batches are made one batch ahead and kept in two.
    const unsigned batch_tiles = 1u << g.az_shift;
    const unsigned batch_lead = batch_tiles == 1 ? 2u : 1u;
    const unsigned batch_buffers = batch_tiles == 1 ? 3u : 2u;
    auto point_data = [&](unsigned n, unsigned s) -> T* { // point s of this workgroup's n-th tile
        const unsigned slot = (((n >> g.az_shift) % batch_buffers) << g.az_shift) | (n & (batch_tiles - 1u));
        return lds + g.off_pts + (slot * S + s) * point_stride;
    };
    auto iterates = [&](unsigned buffer, unsigned s, unsigned which, int l) -> T* {
        return lds + g.off_iter + ((buffer * S + s) * ARRAYS + which) * tri_all + l * (l + 1) / 2;
    };

    // same XCD-contiguous walk as the closed-form kernel
    const unsigned xcd = blockIdx.x & 7u;
    const unsigned rank_in_xcd = blockIdx.x >> 3;
    const unsigned groups_per_xcd = gridDim.x >> 3;
    const unsigned xcd_first = xcd * g.tiles_per_xcd;
    unsigned xcd_last = xcd_first + g.tiles_per_xcd;
    if (xcd_last > g.n_tiles) xcd_last = g.n_tiles;
    // A workgroup takes chunks of C consecutive tiles; the chunks of an XCD's workgroups lie
    // side by side. Consecutive tiles in one workgroup share the 128-byte lines in which one
    // ends and the next begins (see flush_run); C stays small so that what the XCD writes at any
    // moment remains a compact window.
    const unsigned chunk_mask = (1u << g.chunk_shift) - 1u;
    if (xcd_first + (rank_in_xcd << g.chunk_shift) >= xcd_last) return; // whole workgroup

    // the n-th tile of this workgroup, and how many points it has (0 past the end)
    auto tile_of = [&](unsigned n) -> unsigned {
        return xcd_first + ((((n >> g.chunk_shift) * groups_per_xcd + rank_in_xcd)) << g.chunk_shift) +
               (n & chunk_mask);
    };
    auto valid_in = [&](unsigned n) -> unsigned {
        const unsigned t = tile_of(n);
        if (t >= xcd_last) return 0u;
        const unsigned long long first = static_cast<unsigned long long>(t) * S;
        const unsigned long long left = g.n_samples - first;
        return left < S ? static_cast<unsigned>(left) : S;
    };
    // lane j of wave 0 takes point j % S of tile j / S of a batch (batch_tiles * S <= 64)
    auto fetch = [&](unsigned batch, T& rx, T& ry, T& rz) {
        rx = ry = rz = 0;
        const unsigned n = (batch << g.az_shift) + lane / S;
        const unsigned s = lane % S;
        if (lane < batch_tiles * S && s < valid_in(n)) {
            const T* src = xyz + (static_cast<unsigned long long>(tile_of(n)) * S + s) * 3;
            rx = src[0];
            ry = src[1];
            rz = src[2];
        }
    };
    // stage one of a batch of tiles (wave 0; lane == tid there)
    auto azimuth_stage = [&](unsigned batch, T rx, T ry, T rz) {
        const unsigned n = (batch << g.az_shift) + lane / S;
        const unsigned s = lane % S;
        if (lane < batch_tiles * S && s < valid_in(n)) {
            T* rec = point_data(n, s);
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
            rec[7] = p.x2 + p.y2;
            azimuth_job<T>(p, L, rec + 8, rec + 8 + (L + 1), rec + 8 + 2 * (L + 1));
        }
    };
    // stage two of tile n (waves 1 .. g.sequence_waves)
    auto recursion_stage = [&](unsigned n) {
        const unsigned count = valid_in(n);
        const unsigned per_l = count * ARRAYS;
        const unsigned jobs = per_l * static_cast<unsigned>(L - H);
        for (unsigned j = tid - 64; j < jobs; j += 64 * g.sequence_waves) { // waves 1 .. sequence_waves
            const unsigned step = j / per_l;
            const unsigned rest = j - step * per_l;
            const int l = L - static_cast<int>(step); // longest recursions first
            const unsigned s = rest / ARRAYS;
            const unsigned which = rest - s * ARRAYS;
            const T* rec = point_data(n, s);
            sequence_job<T>(l, static_cast<int>(which), rec[2], rec[7], Q, rec + 8 + 2 * (L + 1),
                            iterates(n & 1u, s, which, l));
        }
    };

    // The waves between the sequence waves and the flush waves compute entries.
    const bool streaming = g.row_buffers == 2;
    const unsigned entry_first_wave = 1 + g.sequence_waves;
    const unsigned entry_end_wave = NT / 64 - (streaming ? g.flush_waves : 0u);
    const unsigned wide_first = 64 * entry_first_wave;
    const unsigned wide_lanes = 64 * (entry_end_wave - entry_first_wave);

    constexpr unsigned LINE = 128u / static_cast<unsigned>(sizeof(T)); // elements per 128-byte line
    // position within its 128-byte line of element `element` of an output array
    auto phase_of = [](const T* array, unsigned long long element) -> unsigned {
        return static_cast<unsigned>((reinterpret_cast<uintptr_t>(array) / sizeof(T) + element) % LINE);
    };

    // Where the rows of tile n start within their staging regions. WHOLE: element 0 of a region
    // stands for the start of the 128-byte line in which the tile's run begins in HBM, so the run
    // itself starts `phase` elements in. WHOLE == false: position within 16 bytes of the first
    // staged row, see row_stride. VJP: the rows never leave LDS, no position to match.
    struct Phases {
        unsigned sph, dsph, ddsph;
    };
    auto phases_of = [&](unsigned n) -> Phases {
        const unsigned long long first_point = static_cast<unsigned long long>(tile_of(n)) * S;
        Phases ph;
        ph.sph = VJP ? 0u : phase_of(sph, first_point * ny + skip) % (WHOLE ? LINE : W16);
        ph.dsph = VJP || MODE < 1 ? 0u : phase_of(dsph, first_point * 3 * ny + skip) % (WHOLE ? LINE : W16);
        ph.ddsph = WHOLE && !VJP && MODE == 2 ? phase_of(ddsph, first_point * 9 * ny) : 0u;
        return ph;
    };

    // WHOLE: the closed forms of tile n, one lane per point, into row buffer `buffer`. The
    // entries of a point are cut in slices (by l), dealt to `among` waves of which this is number
    // `who`, so that no single wave carries all of the chain rule and staging.
    auto closed_stage = [&](unsigned n, unsigned buffer, unsigned who, unsigned among) {
        if constexpr (WHOLE) {
            const unsigned valid = valid_in(n);
            if (lane < valid) {
                T* staged = lds + buffer * g.rows_elems;
                const Phases ph = phases_of(n);
                const T* rec = point_data(n, lane);
                Point<T> p;
                p.x = rec[0];
                p.y = rec[1];
                p.z = rec[2];
                p.x2 = rec[3];
                p.y2 = rec[4];
                p.z2 = rec[5];
                p.ir = rec[6];
                Rows<T> rows;
                rows.ny = static_cast<int>(ny);
                rows.sph = staged + ph.sph + lane * ny;
                rows.dsph = staged + g.off_dsph + ph.dsph + lane * 3 * ny;
                rows.ddsph = staged + g.off_ddsph + ph.ddsph + lane * 9 * ny;
                if constexpr (H == 6) {
                    // float32 rows a multiple of 32 words long (l_max = 7, 15, 23, ...): the
                    // stores of all lanes would fall on one LDS bank; stored in rotated fours
                    // instead (closed_form_job; l_max = 7, 500k points, gradients: 343 -> 216 us).
                    // Not for float64 and not for values alone, where the selects cost registers
                    // that the kernel does not have to spare (values: 68 -> 89, and l_max = 9 lost
                    // its third workgroup per CU, 80 -> 106 us).
                    constexpr bool MAY_ROTATE = sizeof(T) == 4 && MODE == 1;
                    if (MAY_ROTATE && (ny & 31u) == 0) {
                        const unsigned turn = lane & 3u;
                        if (0 % among == who) closed_form_job<T, MODE, NORM, H, 0, 8, true>(p, rows, turn);
                        if (1 % among == who) closed_form_job<T, MODE, NORM, H, 8, 16, true>(p, rows, turn);
                        if (2 % among == who) closed_form_job<T, MODE, NORM, H, 16, 24, true>(p, rows, turn);
                        if (3 % among == who) closed_form_job<T, MODE, NORM, H, 24, 32, true>(p, rows, turn);
                        if (4 % among == who) closed_form_job<T, MODE, NORM, H, 32, 40, true>(p, rows, turn);
                        if (5 % among == who) closed_form_job<T, MODE, NORM, H, 40, 49, true>(p, rows, turn);
                    } else {
                        if (0 % among == who) closed_form_job<T, MODE, NORM, H, 0, 9>(p, rows);
                        if (1 % among == who) closed_form_job<T, MODE, NORM, H, 9, 16>(p, rows);
                        if (2 % among == who) closed_form_job<T, MODE, NORM, H, 16, 25>(p, rows);
                        if (3 % among == who) closed_form_job<T, MODE, NORM, H, 25, 31>(p, rows);
                        if (4 % among == who) closed_form_job<T, MODE, NORM, H, 31, 36>(p, rows);
                        if (5 % among == who) closed_form_job<T, MODE, NORM, H, 36, 41>(p, rows);
                        if (6 % among == who) closed_form_job<T, MODE, NORM, H, 41, 45>(p, rows);
                        if (7 % among == who) closed_form_job<T, MODE, NORM, H, 45, 49>(p, rows);
                    }
                } else {
                    if (who == 0) closed_form_job<T, MODE, NORM, H>(p, rows);
                }
            }
        }
    };

    // stage three of tile n, into row buffer `buffer` (the entry waves)
    auto entry_stage = [&](unsigned n, unsigned buffer) {
        const unsigned valid = valid_in(n);
        T* staged = lds + buffer * g.rows_elems;
        const unsigned t = tid - wide_first;
        const Phases ph = phases_of(n);
        const unsigned phase_sph = ph.sph, phase_dsph = ph.dsph, phase_ddsph = ph.ddsph;
        // One pass takes the jobs of as many points as fit side by side in the wide lanes
        // (of one point, in several rounds, when it has more jobs than there are lanes);
        // what depends on the point only is read once per pass.
        unsigned local = 0, e_first = t;
        if (g.points_per_pass > 1) {
            local = __umulhi(t, g.magic_jobs);
            e_first = t - local * g.jobs_per_point;
        }
        for (unsigned s0 = 0; s0 < valid; s0 += g.points_per_pass) {
            const unsigned s = s0 + local;
            if (s >= valid || local >= g.points_per_pass) continue;
            const T* rec = point_data(n, s);
            Point<T> p;
            p.x = rec[0];
            p.y = rec[1];
            p.z = rec[2];
            p.x2 = rec[3];
            p.y2 = rec[4];
            p.z2 = rec[5];
            p.ir = rec[6];
            const T* c = rec + 8;
            const T* sn = rec + 8 + (L + 1);
            const T* itA = iterates(n & 1u, s, 0, 0);
            const T* itB = iterates(n & 1u, s, MODE >= 1 ? 1 : 0, 0);
            const T* itC = iterates(n & 1u, s, MODE == 2 ? 2 : 0, 0);
            // rows are addressed with the entry's index in the full row; shift the bases when
            // the staged rows start at l = H + 1
            Rows<T> rows;
            rows.ny = static_cast<int>(row_stride);
            rows.sph = staged + phase_sph + s * row_stride - skip;
            rows.dsph = staged + g.off_dsph + phase_dsph + s * 3 * row_stride - skip;
            rows.ddsph = staged + g.off_ddsph + phase_ddsph + s * 9 * row_stride - skip;
            for (unsigned e = e_first; e < g.jobs_per_point; e += wide_lanes) {
                const unsigned packed = job_table[e];
                const int m = static_cast<int>(packed & 0x7fu);
                const int side = static_cast<int>((packed >> 7) & 1u);
                const int l = static_cast<int>((packed >> 8) & 0xffu);
                const int tri = static_cast<int>(packed >> 16);
                entry_job<T, MODE, NORM, SPLIT>(l, m, tri, side, p, F + tri, c, sn, itA + tri,
                                                itB + tri, itC + tri, rows);
            }
        }
    };

    // last stage of tile n: row buffer `buffer` to HBM, by `count` threads of which this is
    // number `ft`. `lone` (a std::integral_constant): the copy of a run is the work of a single
    // wave, which then keeps several LDS loads in flight; with all waves of the workgroup on one
    // run, loads and stores alternating one by one measured faster.
    auto flush_stage = [&](unsigned n, unsigned buffer, unsigned ft, unsigned count, auto lone) {
        constexpr int WHOLE_UNROLL = decltype(lone)::value ? SPHX_FLUSH_UNROLL : 1;
        const unsigned valid = valid_in(n);
        const unsigned long long first = static_cast<unsigned long long>(tile_of(n)) * S;
        const T* staged = lds + buffer * g.rows_elems;
        if constexpr (WHOLE) {
            // The tile's run of `len` elements of one output array starts at element `at` of that
            // array. Only whole 128-byte lines go out with vector stores. The line in which the
            // run ends is completed by the next tile: when that tile is this workgroup's next one
            // (same chunk), the unfinished part is carried over into the region the next tile is
            // staged in; at the ends of a chunk the partial lines are stored element by element.
            const bool starts = (n & chunk_mask) == 0;
            const bool ends = (n & chunk_mask) == chunk_mask || valid_in(n + 1) == 0;
            T* carry_to = lds + (streaming ? (buffer ^ 1u) : buffer) * g.rows_elems;
            auto flush_run = [&](unsigned region_offset, T* array, unsigned long long at, unsigned len) {
                using V = typename Pack<T>::type;
                constexpr unsigned W = Pack<T>::width;
                T* region = lds + buffer * g.rows_elems + region_offset;
                const unsigned phase = phase_of(array, at);
                T* line0 = array + (at - phase); // HBM address of region element 0
                const unsigned lo = starts ? phase : 0u; // first element that holds data
                const unsigned hi = phase + len;
                const unsigned full_lo = (lo + LINE - 1u) / LINE * LINE;
                const unsigned full_hi = hi / LINE * LINE;
                unsigned tail_from; // what follows the head and the whole lines
                if (full_hi > full_lo) {
                    const unsigned nvec = (full_hi - full_lo) / W;
                    const V* in = reinterpret_cast<const V*>(region + full_lo);
                    V* out = reinterpret_cast<V*>(line0 + full_lo);
                    unsigned v = ft;
                    if constexpr (WHOLE_UNROLL > 1) {
                        for (; v + (WHOLE_UNROLL - 1) * count < nvec; v += WHOLE_UNROLL * count) {
                            V hold[WHOLE_UNROLL];
#pragma unroll
                            for (int u = 0; u < WHOLE_UNROLL; ++u) hold[u] = in[v + u * count];
#pragma unroll
                            for (int u = 0; u < WHOLE_UNROLL; ++u) {
                                emit<T, SPHX_STREAMING_STORES>(hold[u], out + v + u * count);
                            }
                        }
                    }
                    for (; v < nvec; v += count) {
                        emit<T, SPHX_STREAMING_STORES>(in[v], out + v);
                    }
                    tail_from = full_hi;
                } else {
                    tail_from = full_lo < hi ? full_lo : hi;
                }
                // head: the part of the first line that belongs to this chunk
                const unsigned head_end = full_lo < hi ? full_lo : hi;
                if (lo + ft < head_end) line0[lo + ft] = region[lo + ft];
                // tail: stored if the chunk ends here, else handed to the next tile
                const unsigned tail = hi - tail_from;
                if (ft < tail) {
                    const T value = region[tail_from + ft];
                    if (ends) {
                        line0[tail_from + ft] = value;
                    } else if (carry_to + region_offset != region || tail_from != 0) {
                        carry_to[region_offset + ft] = value;
                    }
                }
            };
            flush_run(0, sph, first * ny, valid * ny);
            if constexpr (MODE >= 1) flush_run(g.off_dsph, dsph, first * 3 * ny, valid * 3 * ny);
            if constexpr (MODE == 2) flush_run(g.off_ddsph, ddsph, first * 9 * ny, valid * 9 * ny);
        } else {
            // one run per (point, component) row, dealt to the waves in turn
            const unsigned waves = count / 64;
            for (unsigned r = ft >> 6; r < valid * components_of(MODE); r += waves) {
                // rows [0, valid) are values, the next 3 * valid are gradients
                if (r < valid) {
                    copy_out<T, SPHX_STREAMING_STORES, false, SPHX_FLUSH_UNROLL>(
                        staged + phase_of(sph, first * ny + skip) % W16 + r * row_stride,
                        sph + (first + r) * ny + skip, nrow, nrow, 0, 0, ft & 63u, 64);
                } else {
                    const unsigned q = r - valid;
                    copy_out<T, SPHX_STREAMING_STORES, false, SPHX_FLUSH_UNROLL>(
                        staged + g.off_dsph + phase_of(dsph, first * 3 * ny + skip) % W16 + q * row_stride,
                        dsph + (first * 3 + q) * ny + skip, nrow, nrow, 0, 0, ft & 63u, 64);
                }
            }
        }
    };

    // VJP: in place of the flush. `sph` holds the upstream gradient sph_grad[N][ny] (read
    // only), `dsph` is xyz_grad[N][3]. Wave 1 + r takes gradient row r of the tile (point r / 3,
    // component r % 3): its lanes multiply the staged entries with the point's row of sph_grad
    // and a butterfly adds the lanes' sums up. With WHOLE == false the staged rows begin at
    // l = H + 1 and closed_form_vjp_kernel has already stored the sum over l <= H, so the
    // result is added to what xyz_grad holds. Wave 0 stays out: it has loads in flight.
    auto contract_stage = [&](unsigned n, unsigned buffer) {
        if constexpr (VJP) {
            const unsigned valid = valid_in(n);
            const unsigned long long first = static_cast<unsigned long long>(tile_of(n)) * S;
            const T* staged = lds + buffer * g.rows_elems + g.off_dsph;
            const T* upstream = sph;
            T* xyz_grad = dsph;
            if (wave == 0) return;
            for (unsigned r = wave - 1; r < valid * 3; r += NT / 64 - 1) {
                const unsigned s = r / 3;
                const T* row = staged + r * row_stride - skip; // indexed with the entry's index in the full row
                const T* weight = upstream + (first + s) * ny;
                T partial = 0;
#pragma unroll 4
                for (unsigned k = skip + lane; k < ny; k += 64) {
                    partial += row[k] * weight[k];
                }
                for (unsigned offset = 32; offset > 0; offset >>= 1) {
                    partial += __shfl_xor(partial, static_cast<int>(offset));
                }
                if (lane == 0) {
                    T* out = xyz_grad + first * 3 + r;
                    *out = (!WHOLE || g.vjp_accumulate) ? *out + partial : partial;
                }
            }
        }
    };

    // fill the pipeline: tables of tiles 0 and 1, iterates of tile 0
    T rx = 0, ry = 0, rz = 0;
    if (wave == 0) {
        fetch(0, rx, ry, rz);
        azimuth_stage(0, rx, ry, rz);
        fetch(1, rx, ry, rz);
    }
    __syncthreads(); // prefactor tables, job table, tables of batch 0
    if (wave == 0) {
        if (batch_lead == 2) {
            azimuth_stage(1, rx, ry, rz);
            fetch(2, rx, ry, rz);
        }
    } else if (wave < entry_first_wave) {
        recursion_stage(0);
    }

    if (streaming) {
        // Two row buffers: while the entry waves fill one with tile n, the flush waves send the
        // other, tile n - 1, to HBM; one barrier per tile, and the stores never pause for the
        // arithmetic. One more round after the last tile flushes it.
        for (unsigned n = 0;; ++n) {
            __syncthreads(); // tables of tile n+1, iterates of tile n, rows of tile n-1 complete
            const unsigned valid = valid_in(n);
            const unsigned before = n > 0 ? valid_in(n - 1) : 0u;
            if (valid == 0 && before == 0) break;
            if (wave == 0) {
                if ((n & (batch_tiles - 1u)) == 0) {
                    azimuth_stage((n >> g.az_shift) + batch_lead, rx, ry, rz);
                    fetch((n >> g.az_shift) + batch_lead + 1, rx, ry, rz); // for the next batch
                }
            } else if (wave < entry_first_wave) {
                recursion_stage(n + 1);
            } else if (wave < entry_end_wave) {
                if (valid != 0) {
                    closed_stage(n, n & 1u, wave - entry_first_wave, entry_end_wave - entry_first_wave);
                    entry_stage(n, n & 1u);
                }
            } else if (before != 0) {
                flush_stage(n - 1, (n - 1) & 1u, tid - 64 * entry_end_wave, 64 * g.flush_waves,
                            std::true_type{});
            }
        }
    } else {
        // One row buffer (the rows of one point fill most of LDS): every wave takes part in the
        // flush, after a second barrier.
        for (unsigned n = 0; valid_in(n) != 0; ++n) {
            __syncthreads(); // tables of tile n+1, iterates of tile n in place; rows of tile n-1 flushed
            // the closed-form slices go round all waves: those that make tables and iterates
            // have time to spare
            closed_stage(n, 0, wave, NT / 64);
            if (wave == 0) {
                if ((n & (batch_tiles - 1u)) == 0) {
                    azimuth_stage((n >> g.az_shift) + batch_lead, rx, ry, rz);
                    fetch((n >> g.az_shift) + batch_lead + 1, rx, ry, rz);
                }
            } else if (wave < entry_first_wave) {
                recursion_stage(n + 1);
            } else {
                entry_stage(n, 0);
            }
            __syncthreads(); // rows of tile n complete
            if constexpr (VJP) {
                contract_stage(n, 0);
            } else {
                flush_stage(n, 0, tid, NT, std::false_type{});
            }
        }
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

struct Launch {
    Tiling g;
    unsigned workgroups;
    unsigned threads;
    unsigned lds_bytes;
};

struct Plan {
    bool lanes;       // values only, short rows: one launch of values_kernel (uses `closed`)
    bool closed_only; // l_max within the closed forms: one launch of closed_form_kernel
    bool whole;       // recursion_kernel evaluates the closed forms too: one launch
                      // otherwise closed_form_kernel<PREFIX> + recursion_kernel: two launches
    bool split_sides; // recursion_kernel takes the entries (l, +m) and (l, -m) as two jobs
    Launch closed;
    Launch rec;
};

static unsigned pow2_floor(unsigned v) {
    unsigned p = 1;
    while (2 * p <= v) p *= 2;
    return p;
}

static unsigned align4(unsigned v) { return (v + 3u) & ~3u; }

static void plan_closed(size_t n_samples, int l_max, int hard, int mode, size_t elem, Launch* out) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = (l_max + 1) * (l_max + 1);
    g.tile = 64;
    g.n_tiles = static_cast<unsigned>((n_samples + 63) / 64);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    out->workgroups = g.tiles_per_xcd * 8u;
    out->threads = 64;
    const unsigned nyh = static_cast<unsigned>(hard + 1) * (hard + 1);
    const unsigned pad = closed_form_pad(hard);
    const unsigned per = 64 / closed_form_phases(static_cast<unsigned>(elem), mode, hard);
    unsigned at = align4(per * (nyh + pad));
    if (mode >= 1) at = align4(at + per * (3 * nyh + pad));
    if (mode == 2) at = align4(at + per * (9 * nyh + pad));
    out->lds_bytes = at * static_cast<unsigned>(elem);
}

// values_kernel: 64 (or 32) points per workgroup, their rows and tables in LDS. Returns false
// when that does not fit, and the recursion kernel takes over.
static bool plan_values(size_t n_samples, int l_max, size_t elem, int lds_limit, Launch* out,
                        bool with_sums = false) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    // rows a multiple of 8 words long: one vector between them (values_kernel)
    const unsigned row_stride = (ny * (esize / 4u)) % 8u == 0 ? ny + vec : ny;
    const unsigned table_stride = (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned tri_all = static_cast<unsigned>(l_max + 1) * (l_max + 2) / 2;
    unsigned allowed = static_cast<unsigned>(env_int("SPHX_VALUES_LDS", 160 * 1024));
    if (allowed > static_cast<unsigned>(lds_limit)) allowed = static_cast<unsigned>(lds_limit);
    // Fewer than 64 points per workgroup leave lanes idle: with 32 the values kernel still beats
    // the recursion kernel (l_max = 32 float32, 500k points: 781 against 1 077 us; l_max = 20
    // float64: 470 against 710), with 16 it does not (l_max = 28 float64: 1 404 against 1 089).
    // The product keeps no rows for HBM in LDS and has far more arithmetic per point to win:
    // it goes down to 8 points (l_max = 24 float64, 200k points: 830 us with 16 points per
    // workgroup against 1 456 us through the recursion kernel).
    const unsigned smallest = static_cast<unsigned>(
        with_sums ? env_int("SPHX_VJP_MIN_TILE", 8) : env_int("SPHX_VALUES_MIN_TILE", 32));
    // Two workgroups per CU (80 KB each) overlap one's tables and flush with the other's
    // arithmetic: preferred, also at half the lanes, over one workgroup with all of LDS
    // (l_max = 16 float32, 500k points: 142 against 164 us; l_max = 12 float64: 115 against 146).
    unsigned tile = 0, rows = 0, bytes = 0;
    for (unsigned limit : {allowed < 80u * 1024u ? allowed : 80u * 1024u, allowed}) {
        for (unsigned t = 64; t >= smallest && t >= 8 && tile == 0; t /= 2) {
            rows = (t * row_stride + vec - 1u) / vec * vec;
            // the product: the waves' sums; with fewer than 64 points also copies of the
            // prefactor tables (vjp_groups_kernel)
            const unsigned extra = !with_sums ? 0u : (t == 64 ? 8u * 3u * 64u : 8u * 3u * 64u + 2u * tri_all);
            bytes = (rows + t * table_stride + extra) * esize;
            if (bytes <= limit) tile = t;
        }
    }
    if (tile == 0) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    if ((n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = row_stride;
    g.off_pts = rows;
    g.off_iter = table_stride;
    g.off_jobs = rows + tile * table_stride; // the product: the waves' sums,
    g.off_F = g.off_jobs + 8u * 3u * 64u;    // and (fewer than 64 points) the prefactor tables
    g.off_Q = g.off_F + tri_all;
    out->workgroups = g.tiles_per_xcd * 8u;
    // one wave per l channel above the closed forms, eight at most
    int waves = env_int("SPHX_VALUES_WAVES", 8);
    waves = waves < 1 ? 1 : (waves > 8 ? 8 : waves);
    // (the product's closed-form slices want at least four; values: one for the tables, one for
    // the closed forms)
    int want = l_max - 6;
    if (with_sums && want < 4) want = 4;
    if (!with_sums && want < 2) want = env_int("SPHX_VALUES_MIN_WAVES", 2);
    out->threads = 64u * static_cast<unsigned>(want < waves ? want : waves);
    out->lds_bytes = bytes;
    return true;
}

// gradients_lanes_kernel: 64, 32 or 16 points per workgroup with their four rows and tables in
// LDS. Returns false when too few points would be resident on a CU for it to pay.
static bool plan_gradient_lanes(size_t n_samples, int l_max, size_t elem, int lds_limit, Launch* out) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    auto stride_of = [&](unsigned block) { return (block * (esize / 4u)) % 8u == 0 ? block + vec : block; };
    const unsigned s_stride = stride_of(ny), d_stride = stride_of(3u * ny);
    const unsigned table_stride = (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned limit = static_cast<unsigned>(lds_limit);
    // Which tile: the one that keeps most points resident on a CU (tile times the workgroups
    // that fit), a tile of 16 counted at three quarters because it leaves three lanes in four
    // idle; between equals the larger tile, unless its workgroup would be alone on the CU (two
    // overlap one another's phases). Measured, 500k points, float32: l_max = 7 105 us with
    // 2 x 64 points against 119 with 4 x 32; l_max = 9 173 us with 2 x 32 against 186 with 64;
    // l_max = 13 357 us with 3 x 16 against 433 with 32; l_max = 15 579 us with 32 against 651
    // with 2 x 16. Below 32 resident points (or 3 x 16) the recursion kernel is the faster one
    // (l_max = 18: 1 038 us against 1 236).
    unsigned tile = 0, off_d = 0, off_t = 0, bytes = 0, best = 0, best_groups = 0;
    for (unsigned t = 64; t >= 16; t /= 2) {
        const unsigned od = (t * s_stride + vec - 1u) / vec * vec;
        const unsigned ot = od + (t * d_stride + vec - 1u) / vec * vec;
        const unsigned b = (ot + t * table_stride) * esize;
        if (b > limit) continue;
        unsigned score = (limit / b) * t * (t >= 32 ? 4u : 3u);
        if (static_cast<unsigned>(env_int("SPHX_GRADIENT_LANES_TILE", 0)) == t) score = 1u << 30;
        if (score > best || (score == best && best_groups < 2)) {
            best = score;
            best_groups = limit / b;
            tile = t;
            off_d = od;
            off_t = ot;
            bytes = b;
        }
    }
    if (best < 32u * 4u) tile = 0;
    if (tile == 0 || (n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = s_stride;
    g.off_dsph = off_d;
    g.off_ddsph = d_stride;
    g.off_pts = off_t;
    g.off_iter = table_stride;
    out->workgroups = g.tiles_per_xcd * 8u;
    int waves = env_int("SPHX_GRADIENT_LANES_WAVES", 8);
    waves = waves < 1 ? 1 : (waves > 8 ? 8 : waves);
    out->threads = 64u * static_cast<unsigned>(waves);
    out->lds_bytes = bytes;
    return true;
}

// hessians_lanes_kernel: 64 or 32 points per workgroup with their thirteen rows, tables and
// iterates in LDS. Returns false when 32 points do not fit.
static bool plan_hessian_lanes(size_t n_samples, int l_max, size_t elem, int lds_limit, Launch* out) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned vec = 16u / esize;
    auto stride_of = [&](unsigned block) { return (block * (esize / 4u)) % 8u == 0 ? block + vec : block; };
    const unsigned s_stride = stride_of(ny), d_stride = stride_of(3u * ny), dd_stride = stride_of(9u * ny);
    const unsigned table_stride = (3u * static_cast<unsigned>(l_max + 1)) | 1u;
    const unsigned channels = static_cast<unsigned>(l_max - 1);
    const unsigned most = kHessianLaneThreads / 64u;
    const unsigned waves = channels < most ? channels : most;
    const unsigned limit = static_cast<unsigned>(lds_limit);
    unsigned tile = 0, off_d = 0, off_dd = 0, off_t = 0, off_s = 0, bytes = 0, best = 0, best_groups = 0;
    for (unsigned t = 64; t >= 32; t /= 2) {
        const unsigned od = (t * s_stride + vec - 1u) / vec * vec;
        const unsigned odd = od + (t * d_stride + vec - 1u) / vec * vec;
        const unsigned ot = odd + (t * dd_stride + vec - 1u) / vec * vec;
        const unsigned os = ot + t * table_stride;
        const unsigned b = (os + waves * t * table_stride) * esize;
        if (b > limit) continue;
        const unsigned score = (limit / b) * t;
        if (score > best || (score == best && best_groups < 2)) {
            best = score;
            best_groups = limit / b;
            tile = t;
            off_d = od;
            off_dd = odd;
            off_t = ot;
            off_s = os;
            bytes = b;
        }
    }
    if (tile == 0 || (n_samples + tile - 1) / tile > 0x7fffffffull) return false;
    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(tile);
    g.n_tiles = static_cast<unsigned>((n_samples + tile - 1) / tile);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    g.rows_elems = s_stride;
    g.off_dsph = d_stride;
    g.off_ddsph = dd_stride;
    g.off_F = off_d;
    g.off_Q = off_dd;
    g.off_pts = off_t;
    g.off_iter = table_stride;
    g.off_jobs = off_s;
    g.jobs_per_point = table_stride;
    out->workgroups = g.tiles_per_xcd * 8u;
    out->threads = 64u * waves;
    out->lds_bytes = bytes;
    return true;
}

// Tile size and LDS layout of the recursion kernel. Returns false when not even one point fits.
static bool plan_recursion(size_t n_samples, int l_max, int mode, bool whole, size_t elem,
                           unsigned budget, int lds_limit, int cus, Launch* out, bool* split_sides) {
    Tiling& g = out->g;
    std::memset(&g, 0, sizeof(g));
    const int hard = mode == 2 ? 1 : 6;
    const unsigned esize = static_cast<unsigned>(elem);
    const unsigned ny = static_cast<unsigned>(l_max + 1) * (l_max + 1);
    const unsigned nyh = static_cast<unsigned>(hard + 1) * (hard + 1);
    const unsigned nrow = whole ? ny : ny - nyh;
    const unsigned tri_all = static_cast<unsigned>(l_max + 1) * (l_max + 2) / 2;
    const unsigned arrays = mode + 1;
    unsigned jobs = 0;
    for (int l = hard + 1; l <= l_max; ++l) jobs += l + 1;
    // with the sides split every (l, m > 0) pair is two jobs; the job table is sized for that
    const unsigned jobs_split = 2 * jobs - static_cast<unsigned>(l_max - hard);
    bool may_split = mode == 2 && env_int("SPHX_SPLIT_SIDES", 1) != 0;
    auto table_elems_for = [&](bool split) { return ((split ? jobs_split : jobs) * 4 + esize - 1) / esize; };
    // per point: the rows in every row buffer, point tables three times, iterates twice
    // staged rows are `row_stride` apart (recursion_kernel): nrow, or a little more when the rows
    // are cut so that they keep their position within 16 bytes
    const unsigned row_stride = nrow + (whole ? 0u : nyh % (16u / esize));
    const unsigned rows_per_point = components_of(mode) * row_stride;
    const unsigned rest_per_point = 3 * (8 + 3 * (l_max + 1)) + 2 * arrays * tri_all;
    unsigned fixed = 0;
    auto bytes_for = [&](unsigned S, unsigned buffers) {
        return (S * (buffers * rows_per_point + rest_per_point) + fixed) * esize;
    };
    const unsigned limit = static_cast<unsigned>(lds_limit);
    for (;;) {
        // 24: alignment slack of the row arrays
        // + 3 lines: a staging region starts at a line boundary of its output array
        fixed = 2 * tri_all + table_elems_for(may_split) + 24 + 2 * 3 * (128u / esize);
        if (bytes_for(1, 1) <= limit || !may_split) break;
        may_split = false; // the longer job table is what does not fit
    }
    // Two row buffers (tile n flushed by a wave of its own while tile n+1 is computed) pay off
    // where the rows of a point are so long that a single buffer holds one or two points and
    // the flush of such a tile is long: measured with second derivatives (l_max = 16, float64:
    // 770 us against 810 us). With many points per tile, or with the rows cut in two kernels,
    // one buffer flushed by all waves measured faster.
    int want_buffers = env_int("SPHX_ROW_BUFFERS", 0);
    if (want_buffers == 0) {
        const unsigned single = bytes_for(1, 1) <= budget
                                    ? (budget / esize - fixed) / (rows_per_point + rest_per_point)
                                    : 1u;
        want_buffers = mode == 2 && single <= 2 ? 2 : 1;
    }
    unsigned buffers = want_buffers == 2 ? 2u : 1u;
    if (bytes_for(1, buffers) > limit) buffers = 1;
    if (bytes_for(1, buffers) > limit) return false;
    unsigned S = 1;
    if (bytes_for(1, buffers) <= budget) {
        S = pow2_floor((budget / esize - fixed) / (buffers * rows_per_point + rest_per_point));
        if (S > 64) S = 64;
    }
    const int forced = env_int("SPHX_TILE", 0);
    if (forced > 0 && forced <= 64 && bytes_for(forced, buffers) <= limit) {
        S = static_cast<unsigned>(forced);
    }

    // Point tables for several tiles at a time (recursion_kernel, az_shift): as many tiles as
    // wave 0 has lanes for, eight at most, as long as the larger table area keeps the workgroup
    // within the budget (or within what it needs anyway).
    const unsigned point_record = 8 + 3 * static_cast<unsigned>(l_max + 1);
    unsigned az_shift = 0;
    {
        const unsigned allowed = bytes_for(S, buffers) > budget ? bytes_for(S, buffers) : budget;
        const int cap = env_int("SPHX_AZ_SHIFT", 3);
        for (unsigned shift = cap < 0 ? 0u : (cap > 6 ? 6u : static_cast<unsigned>(cap)); shift >= 1; --shift) {
            const unsigned tiles = 1u << shift;
            if (tiles * S > 64) continue;
            const unsigned extra = (2 * tiles - 3) * S * point_record * esize;
            if (bytes_for(S, buffers) + extra <= allowed || bytes_for(S, buffers) + extra <= budget) {
                az_shift = shift;
                break;
            }
        }
    }
    const unsigned table_slots = az_shift == 0 ? 3u : 2u << az_shift;

    g.n_samples = n_samples;
    g.l_max = l_max;
    g.ny = static_cast<int>(ny);
    g.tile = static_cast<int>(S);
    g.az_shift = az_shift;
    g.row_buffers = buffers;
    g.flush_waves = buffers == 2 ? static_cast<unsigned>(env_int("SPHX_FLUSH_WAVES", 1)) : 0u;
    if (g.flush_waves > 2) g.flush_waves = 2;
    if (buffers == 2 && g.flush_waves < 1) g.flush_waves = 1;
    g.sequence_waves = S * arrays * static_cast<unsigned>(l_max - hard) > 64 ? 2u : 1u;
    // Split the sides when that lets the entries of a tile go through the entry waves in fewer
    // rounds than it costs: a one-sided job is about 0.6 of a two-sided one.
    const unsigned wide = kRecursionThreads - 64 * (1 + g.sequence_waves + g.flush_waves);
    auto per_pass = [&](unsigned j) { return j >= wide ? 1u : wide / j; };
    auto rounds = [&](unsigned j) {
        return ((S + per_pass(j) - 1) / per_pass(j)) * ((j + wide - 1) / wide);
    };
    *split_sides = may_split && 6 * rounds(jobs_split) < 10 * rounds(jobs);
    g.jobs_per_point = *split_sides ? jobs_split : jobs;
    g.magic_jobs = magic_of(g.jobs_per_point);
    g.points_per_pass = per_pass(g.jobs_per_point);

    // in front of every staging region, room for the part of a 128-byte line that precedes the
    // tile's run (recursion_kernel, flush_run)
    const unsigned line = whole ? 128u / esize : 16u / esize;
    unsigned at = align4(S * row_stride + line);
    g.off_dsph = at;
    if (mode >= 1) at = align4(at + S * 3 * row_stride + line);
    g.off_ddsph = at;
    if (mode == 2) at = align4(at + S * 9 * row_stride + line);
    g.rows_elems = at;
    at *= buffers;
    g.off_F = at;
    at += tri_all;
    g.off_Q = at;
    at += tri_all;
    g.off_pts = at;
    at += table_slots * S * point_record;
    g.off_iter = at;
    at += 2 * S * arrays * tri_all;
    g.off_jobs = at;
    at += table_elems_for(may_split);
    out->lds_bytes = at * esize;
    out->threads = kRecursionThreads;
    if (out->lds_bytes > limit) return false;

    g.n_tiles = static_cast<unsigned>((n_samples + S - 1) / S);
    g.tiles_per_xcd = (g.n_tiles + 7u) / 8u;
    // Chunks of consecutive tiles per workgroup: only where a tile is one run per array, and a
    // run is at least a line long (so that a carried part never spans two tiles).
    g.chunk_shift = 0;
    if (whole && S * nrow * esize >= 128u) {
        const int want = env_int("SPHX_CHUNK_SHIFT", 3);
        g.chunk_shift = want < 0 ? 0u : (want > 10 ? 10u : static_cast<unsigned>(want));
    }
    unsigned per_cu = limit / out->lds_bytes;
    if (per_cu < 1) per_cu = 1;
    if (per_cu > 4) per_cu = 4; // 512 threads each: 2048 lanes per CU
    unsigned want = (static_cast<unsigned>(cus) * per_cu + 7u) & ~7u;
    // Few points: shorter chunks, down to single tiles, until every resident workgroup has one
    // (10 000 points at l_max = 8 are 625 tiles of 16: in chunks of 8 they kept 80 workgroups
    // busy for 41 us, as single tiles they take 512 and a third of the time).
    auto chunks_in_xcd = [&]() { return (g.tiles_per_xcd + (1u << g.chunk_shift) - 1u) >> g.chunk_shift; };
    while (g.chunk_shift > 0 && chunks_in_xcd() * 8u < want) --g.chunk_shift;
    const unsigned chunks_per_xcd = chunks_in_xcd();
    unsigned need = chunks_per_xcd * 8u;
    out->workgroups = want < need ? want : need;
    if (out->workgroups < 8) out->workgroups = 8;
    return true;
}

// Choose kernels, tile sizes and LDS layouts. `lds_limit` / `cus` describe the device.
static int make_plan(size_t n_samples, int l_max, int mode, size_t elem, int lds_limit, int cus,
                     Plan* plan, bool lane_kernels = true) {
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (mode < 0 || mode > 2) return fail(SPHX_ERR_ARGUMENT, "unknown derivative selector");
    if (l_max > SPHX_TABLE_LMAX) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) + " exceeds the device prefactor tables (" +
                        std::to_string(SPHX_TABLE_LMAX) + ")");
    }
    if ((n_samples + 63) / 64 > 0x7fffffffull) {
        return fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    }
    const int hard = mode == 2 ? 1 : 6;
    plan->lanes = false;
    plan->closed_only = l_max <= hard;
    plan->whole = true;
    plan->split_sides = false;
    if (plan->closed_only) {
        plan_closed(n_samples, l_max, l_max, mode, elem, &plan->closed);
        return SPHX_OK;
    }
    if (lane_kernels && mode == 0 && plan_values(n_samples, l_max, elem, lds_limit, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    // Second derivatives at small l_max: one point per lane where that was measured to be faster
    // than the recursion kernel (SPHX_HESSIAN_LANES: 0 never, 2 wherever the rows fit).
    const int hessian_lanes = env_int("SPHX_HESSIAN_LANES", 1);
    const bool hessian_lanes_pay = elem == 4 ? (l_max <= 5 || l_max == 7) : l_max <= 5;
    if (lane_kernels && mode == 2 && (hessian_lanes == 2 || (hessian_lanes == 1 && hessian_lanes_pay)) &&
        plan_hessian_lanes(n_samples, l_max, elem, lds_limit, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    if (lane_kernels && mode == 1 && env_int("SPHX_GRADIENT_LANES", 1) != 0 &&
        plan_gradient_lanes(n_samples, l_max, elem, lds_limit, &plan->closed)) {
        plan->lanes = true;
        return SPHX_OK;
    }
    const unsigned budget = static_cast<unsigned>(env_int("SPHX_TILE_LDS_BUDGET", 80 * 1024));
    bool fits = plan_recursion(n_samples, l_max, mode, true, elem, budget, lds_limit, cus, &plan->rec,
                               &plan->split_sides);
    // With very few points per tile the one-lane-per-point closed forms of l <= 6 would leave
    // most of the lanes idle for some two thousand instructions per tile: hand them to the
    // closed-form kernel, which runs them 64 points at a time, and let the recursion kernel stage
    // l >= 7 only. The price is rows cut in two, each part a run of its own in HBM, so the
    // threshold is low (measured, 1M/500k/200k points, gradients: float32 l_max = 16, 8 points
    // per tile, 812 us whole against 1110 us cut; l_max = 24, 4 points, 593 against 729;
    // float64 l_max = 12, 8 points, 513 against 655; l_max = 20, 2 points, 1801 against 1018).
    const int split_below = env_int("SPHX_SPLIT_BELOW", elem == 4 ? 4 : 8);
    if (mode < 2 && (!fits || plan->rec.g.tile < split_below)) {
        Launch upper;
        if (plan_recursion(n_samples, l_max, mode, false, elem, budget, lds_limit, cus, &upper,
                           &plan->split_sides)) {
            plan->whole = false;
            plan->rec = upper;
            plan_closed(n_samples, l_max, hard, mode, elem, &plan->closed);
            fits = true;
        }
    }
    if (!fits) {
        return fail(SPHX_ERR_UNSUPPORTED,
                    "l_max = " + std::to_string(l_max) +
                        " with this many derivatives needs more LDS for the rows of one point than "
                        "the device offers (" + std::to_string(lds_limit) + " bytes)");
    }
    return SPHX_OK;
}

// What a launch needs to know about a kernel on a device, asked from the runtime once per
// (device, kernel, LDS size) instead of on every call: the calls take microseconds each, which
// is the whole budget of a small evaluation.
struct KernelFacts {
    int device;
    const void* kernel;
    unsigned lds_bytes;
    unsigned resident_workgroups; // on the whole device, a multiple of 8; 0 = unknown
};
static std::mutex g_facts_mutex;
static std::vector<KernelFacts> g_facts;

// Raises the kernel's dynamic LDS limit if needed and returns how many workgroups of `threads`
// threads are resident on the device at once (0 if the runtime would not tell).
static hipError_t kernel_facts(const void* kernel, unsigned threads, unsigned lds_bytes,
                               unsigned* resident_workgroups) {
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e != hipSuccess) return e;
    {
        std::lock_guard<std::mutex> lock(g_facts_mutex);
        for (const KernelFacts& f : g_facts) {
            if (f.device == device && f.kernel == kernel && f.lds_bytes == lds_bytes) {
                *resident_workgroups = f.resident_workgroups;
                return hipSuccess;
            }
        }
    }
    if (lds_bytes > 64u * 1024u) {
        // the limit of the device, not of this launch: the attribute belongs to the kernel, and
        // a later launch with less must not lower it for one with more that is already cached
        int limit = device >= 0 && device < kMaxDevices ? g_lds_limit[device] : 0;
        if (limit < static_cast<int>(lds_bytes)) limit = static_cast<int>(lds_bytes);
        e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, limit);
        if (e != hipSuccess) return e;
    }
    KernelFacts fresh{device, kernel, lds_bytes, 0u};
    int per_cu = 0;
    const int cus = device >= 0 && device < kMaxDevices ? g_compute_units[device] : 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, static_cast<int>(threads),
                                                     lds_bytes) == hipSuccess &&
        per_cu > 0 && cus > 0) {
        fresh.resident_workgroups = (static_cast<unsigned>(per_cu) * static_cast<unsigned>(cus)) & ~7u;
    } else {
        (void)hipGetLastError();
    }
    std::lock_guard<std::mutex> lock(g_facts_mutex);
    g_facts.push_back(fresh);
    *resident_workgroups = fresh.resident_workgroups;
    return hipSuccess;
}

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

template <typename T, int MODE, bool NORM, bool WHOLE, bool SPLIT, bool VJP = false>
static hipError_t launch_recursion(const Launch& l, const T* xyz, T* sph, T* dsph, T* ddsph,
                                   hipStream_t stream) {
    auto kernel = recursion_kernel<T, MODE, NORM, WHOLE, SPLIT, VJP>;
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
static hipError_t dispatch(const Plan& plan, const T* xyz, T* sph, T* dsph, T* ddsph,
                           hipStream_t stream) {
    if (plan.lanes) {
        if constexpr (MODE == 0) {
            const Launch& l = plan.closed;
            auto kernel = values_kernel<T, NORM>;
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
            auto kernel = gradients_lanes_kernel<T, NORM>;
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
static hipError_t dispatch_vjp(const Launch& l, int l_max, const T* xyz, const T* sph_grad,
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
static int vjp(const T* xyz, const T* sph_grad, size_t n_samples, int l_max, int normalized,
               T* xyz_grad, int accumulate, void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
    if (l_max < 0) return fail(SPHX_ERR_ARGUMENT, "l_max must be non-negative");
    if (xyz == nullptr || sph_grad == nullptr || xyz_grad == nullptr) {
        return fail(SPHX_ERR_ARGUMENT, "null pointer passed to the vector-Jacobian product");
    }
    if ((n_samples + 63) / 64 > 0x7fffffffull) {
        return fail(SPHX_ERR_UNSUPPORTED, "too many samples for one launch");
    }
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
    Launch lanes;
    bool use_lanes = false;
    if (status == SPHX_OK) {
        if (l_max > SPHX_TABLE_LMAX) {
            status = fail(SPHX_ERR_UNSUPPORTED, "l_max = " + std::to_string(l_max) +
                                                    " exceeds the device prefactor tables (" +
                                                    std::to_string(SPHX_TABLE_LMAX) + ")");
        } else if (l_max > 6 && env_int("SPHX_VJP_LANES", 1) != 0) {
            use_lanes = plan_values(n_samples, l_max, sizeof(T), g_lds_limit[device], &lanes, true);
        }
    }
    if (status == SPHX_OK && !use_lanes) {
        // the closed-form or the recursion kernels with the contraction in place of the flush
        status = make_plan(n_samples, l_max, 1, sizeof(T), g_lds_limit[device], g_compute_units[device],
                           &plan, false);
    }
    if (status == SPHX_OK) {
        hipStream_t s = reinterpret_cast<hipStream_t>(stream);
        hipError_t e;
        if (use_lanes) {
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
            // groups of lanes with channels of their own pay off from tiles of 16 points down
            // (200k points, float32 l_max = 24: 225 against 279 us; float64 l_max = 24: 665
            // against 866; with tiles of 32 the scalar-unit kernel is ahead, float64 l_max = 12:
            // 329 against 397)
            if (lanes.g.tile > env_int("SPHX_VJP_GROUPS_BELOW", 16)) {
                e = normalized ? launch(vjp_lanes_kernel<T, true>) : launch(vjp_lanes_kernel<T, false>);
            } else {
                e = normalized ? launch(vjp_groups_kernel<T, true>) : launch(vjp_groups_kernel<T, false>);
            }
        } else if (plan.closed_only) {
            e = normalized ? dispatch_vjp<T, true>(plan.closed, l_max, xyz, sph_grad, xyz_grad, accumulate, s)
                           : dispatch_vjp<T, false>(plan.closed, l_max, xyz, sph_grad, xyz_grad, accumulate, s);
        } else {
            e = normalized ? launch_vjp_recursion<T, true>(plan, xyz, sph_grad, xyz_grad, accumulate, s)
                           : launch_vjp_recursion<T, false>(plan, xyz, sph_grad, xyz_grad, accumulate, s);
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

// ---------------------------------------------------------------------------
// float32 arrays evaluated in float64. In float32 the reference's prefactors
// and Q_l^l = (2l-1)!! leave the range of the type from l = 29 (NaN and inf in
// the outputs) and high-|m| entries come out as exact zeros from l of about 20
// (sphericart/include/templates.hpp:54-97 evaluated in float). This path, which
// a caller must ask for, widens xyz, runs the float64 kernels into a workspace
// and rounds every result once.
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

static int forward_f32_via_f64(const float* xyz, size_t n_samples, int l_max, int normalized, int mode,
                               float* sph, float* dsph, float* ddsph, void* workspace,
                               size_t workspace_bytes, void* stream) {
    t_error.clear();
    if (n_samples == 0) return SPHX_OK;
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

    hipPointerAttribute_t attr;
    SPHX_HIP(hipPointerGetAttributes(&attr, xyz));
    int current = 0;
    SPHX_HIP(hipGetDevice(&current));
    const int device = attr.device;
    if (device != current) SPHX_HIP(hipSetDevice(device));

    const size_t per_point = via_f64_bytes_per_point(l_max, mode);
    const size_t ny = static_cast<size_t>(l_max + 1) * (l_max + 1);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    int status = SPHX_OK;
    void* owned = nullptr;
    if (workspace == nullptr) {
        // no workspace given: one of our own for at most 256 MiB worth of points at a time
        size_t points = (size_t(256) << 20) / per_point;
        if (points < 64) points = 64;
        if (points > n_samples) points = n_samples;
        workspace_bytes = points * per_point;
        hipError_t e = hipMalloc(&owned, workspace_bytes);
        if (e != hipSuccess) {
            status = fail(SPHX_ERR_HIP, std::string("hipMalloc of the float64 workspace: ") + hipGetErrorString(e));
        }
        workspace = owned;
    }
    size_t chunk = workspace_bytes / per_point;
    if (status == SPHX_OK && chunk == 0) {
        status = fail(SPHX_ERR_ARGUMENT, "the workspace holds no point: " + std::to_string(per_point) +
                                             " bytes are needed per point");
    }
    if (status == SPHX_OK && (reinterpret_cast<uintptr_t>(workspace) & 15u) != 0) {
        status = fail(SPHX_ERR_ARGUMENT, "the workspace must be aligned to 16 bytes");
    }
    if (chunk > n_samples) chunk = n_samples;
    if (chunk >= 64) chunk &= ~size_t(63); // whole tiles of the closed-form kernels
    // workspace layout for a chunk of c points: sph[c][ny], dsph[c][3][ny], ddsph[c][9][ny], xyz[c][3]
    double* w_sph = static_cast<double*>(workspace);
    double* w_dsph = w_sph + chunk * ny;
    double* w_ddsph = w_dsph + (mode >= 1 ? chunk * 3 * ny : 0);
    double* w_xyz = w_ddsph + (mode >= 2 ? chunk * 9 * ny : 0);
    for (size_t first = 0; status == SPHX_OK && first < n_samples; first += chunk) {
        const size_t count = n_samples - first < chunk ? n_samples - first : chunk;
        hipLaunchKernelGGL(widen_kernel, dim3(convert_blocks(count * 3)), dim3(kConvertThreads), 0, s,
                           xyz + first * 3, w_xyz, static_cast<unsigned long long>(count * 3));
        status = forward<double>(w_xyz, count, l_max, normalized, mode, w_sph, mode >= 1 ? w_dsph : nullptr,
                                 mode >= 2 ? w_ddsph : nullptr, stream);
        if (status != SPHX_OK) break;
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
            status = fail(SPHX_ERR_HIP, std::string("kernel launch: ") + hipGetErrorString(e));
        }
    }
    if (owned != nullptr) {
        // our own workspace: wait for the work that uses it, then give it back
        hipError_t e = hipStreamSynchronize(s);
        if (e != hipSuccess && status == SPHX_OK) {
            status = fail(SPHX_ERR_HIP, std::string("hipStreamSynchronize: ") + hipGetErrorString(e));
        }
        e = hipFree(owned);
        if (e != hipSuccess && status == SPHX_OK) {
            status = fail(SPHX_ERR_HIP, std::string("hipFree: ") + hipGetErrorString(e));
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

int sphx_forward_f32_via_f64(const float* xyz, size_t n_samples, int l_max, int normalized,
                             int derivatives, float* sph, float* dsph, float* ddsph, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return sphx::forward_f32_via_f64(xyz, n_samples, l_max, normalized, derivatives, sph, dsph, ddsph,
                                     workspace, workspace_bytes, stream);
}

size_t sphx_forward_f32_via_f64_workspace(size_t n_samples, int l_max, int derivatives) {
    if (l_max < 0 || derivatives < 0 || derivatives > 2) return 0;
    return n_samples * sphx::via_f64_bytes_per_point(l_max, derivatives);
}

int sphx_vjp_f32(const float* xyz, const float* sph_grad, size_t n_samples, int l_max, int normalized,
                 float* xyz_grad, int accumulate, void* stream) {
    return sphx::vjp<float>(xyz, sph_grad, n_samples, l_max, normalized, xyz_grad, accumulate, stream);
}

int sphx_vjp_f64(const double* xyz, const double* sph_grad, size_t n_samples, int l_max,
                 int normalized, double* xyz_grad, int accumulate, void* stream) {
    return sphx::vjp<double>(xyz, sph_grad, n_samples, l_max, normalized, xyz_grad, accumulate, stream);
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
    const sphx::Launch& main = plan.closed_only || plan.lanes ? plan.closed : plan.rec;
    if (tile_samples) *tile_samples = main.g.tile;
    if (threads) *threads = static_cast<int>(main.threads);
    if (lds_bytes) *lds_bytes = static_cast<int>(main.lds_bytes);
    if (workgroups) *workgroups = static_cast<int>(main.workgroups);
    return SPHX_OK;
}

} // extern "C"
