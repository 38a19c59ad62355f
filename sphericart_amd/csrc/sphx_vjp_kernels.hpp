// Vector-Jacobian products that never write the Jacobian: closed_form_vjp_kernel (l_max <= 6),
// vjp_lanes_kernel and vjp_groups_kernel (beyond, one point per lane or per lane of a group).
#ifndef SPHX_VJP_KERNELS_HPP
#define SPHX_VJP_KERNELS_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sphx_tiling.hpp"
#include "sphx_closed_form_kernel.hpp"
#include "sphx_lane_kernels.hpp"

namespace sphx {

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
template <typename T, bool NORM, unsigned NT = kValuesMaxThreads>
__global__ __launch_bounds__(NT) void vjp_lanes_kernel(Tiling g, const T* __restrict__ xyz,
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
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same for all lanes: scalar
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
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same for all lanes: scalar
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

} // namespace sphx

#endif
