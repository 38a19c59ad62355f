// One point per lane, l and m the same for a whole wave: values_kernel, gradients_lanes_kernel and
// hessians_lanes_kernel, for the l_max at which the rows of 16 to 64 points fit in LDS.
#ifndef SPHX_LANE_KERNELS_HPP
#define SPHX_LANE_KERNELS_HPP

#include <hip/hip_runtime.h>

#include <cstdint>
#include <type_traits>

#include "sphx_tiling.hpp"

namespace sphx {

// ---------------------------------------------------------------------------
// Values only, l_max > 6, rows short enough that those of 16 to 64 points fit
// in LDS: one point per lane, one to eight waves that share the l channels of
// the same points.
//
// Without derivatives an entry is three multiplications, so what counts is what
// surrounds them. With one point per lane l and m are the same for the whole
// wave: no job has to be decoded and no iterate passes through LDS. The
// prefactors of a channel, m = 0..l, are loaded once, one per lane, and the
// recursion takes each from its lane (v_readlane), so that its loop touches no
// memory but the point's table in LDS, whose entries for the next m are fetched
// before the arithmetic of this one: about 25 instructions per (l, +-m) pair of
// entries, a fraction of what the recursion kernel spends on them. (Prefactors
// through scalar loads inside the loop made every step wait for them: LDS and
// scalar loads share one counter, so nothing could be fetched ahead. 1 GB of
// values, float32, l_max = 22, 26, 28: 288, 341, 355 us then, 270, 315, 327 so.)
// (With derivatives the entries themselves dominate and rows are four and
// thirteen times as long, so that far fewer than 64 points fit:
// gradients_lanes_kernel takes l_max up to about 16, the recursion kernel the
// rest.)
//
// The rows of 64 points take most of a CU's LDS from l_max of about 12 on, and
// one wave would leave three of the four SIMDs idle: the l channels are dealt
// to the waves of the workgroup (in snake order, long and short ones mixed),
// each wave evaluating its channels for all points of the tile (l_max = 15
// float32, 500k points: 245 us with one wave, 113 with four, 106 with six).
// When 64 rows do not fit the tile is smaller, any number of points, and the
// lanes beyond it idle; or (K = 2, 4) the tile is 32 or 16 points and a wave
// evaluates K channels l0, l0 - 1, .. side by side, lane = side * (64 / K) +
// point: it walks m down from l0 for all of them, each lane picks the
// prefactors of its own channel, and the lanes of a shorter channel join when
// m reaches their l. All lanes work then, for about 40 instructions per step
// of two channels (the host picks by shape, see plan_values).
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

// The value a given lane holds, for the whole wave (the lane number is the same for all lanes).
__device__ __forceinline__ float from_lane(float v, int lane) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ double from_lane(double v, int lane) {
    const long long bits = __double_as_longlong(v);
    const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(bits), lane));
    const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<int>(bits >> 32), lane));
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}

// Prefactors of one l channel, m = 0..l: lane j of the wave holds that of m = j (one load for the
// whole channel; all lanes must be active), and the recursion takes them from there with no
// memory access in its loop. For l <= 63.
template <typename T> struct ChannelPrefactors {
    T lanes;
    __device__ __forceinline__ ChannelPrefactors() : lanes(0) {}
    __device__ __forceinline__ ChannelPrefactors(const T* row, int l, unsigned lane)
        : lanes(row[static_cast<int>(lane) < l ? static_cast<int>(lane) : l]) {
        // keeps the load here, where all lanes are active: its only uses are the reads of single
        // lanes, and it would otherwise be moved to them, into code that only some lanes run
        asm volatile("" : "+v"(lanes));
    }
    __device__ __forceinline__ T operator[](int m) const { return from_lane(lanes, m); }
};

template <typename T, bool NORM, unsigned K = 1, unsigned NT = kValuesMaxThreads>
__global__ __launch_bounds__(NT) void values_kernel(Tiling g, const T* __restrict__ xyz,
                                                                  T* __restrict__ sph) {
    constexpr int H = 6;
    constexpr unsigned NYH = (H + 1) * (H + 1);
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    T* lds = reinterpret_cast<T*>(lds_raw);
    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u;
    const unsigned wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same for all lanes: scalar
    const unsigned waves = blockDim.x >> 6;
    const int L = g.l_max;
    const unsigned ny = g.ny;
    const unsigned group = (blockIdx.x & 7u) * g.tiles_per_xcd + (blockIdx.x >> 3);
    if (group >= g.n_tiles) return;
    const unsigned tile = static_cast<unsigned>(g.tile); // 64, or fewer when 64 rows do not fit
    const unsigned long long first = static_cast<unsigned long long>(group) * tile;
    const unsigned long long left = g.n_samples - first;
    const unsigned valid = left < tile ? static_cast<unsigned>(left) : tile;

    // K > 1: the tile is 64 / K points, and lane = side * (64 / K) + point
    const unsigned point = K == 1 ? lane : lane & (64u / K - 1u);
    const unsigned side = K == 1 ? 0u : lane / (64u / K);
    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    T* row = lds + point * g.rows_elems;
    T* tab = lds + g.off_pts + point * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    if (point < valid) p = load_point<T, NORM>(xyz + (first + point) * 3);
    if (point < valid && side == 0) {
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
    if constexpr (K > 1) {
        const T rxy = p.x2 + p.y2;
        // K channels side by side, l0, l0 - 1, ..: the wave walks m from l0 down for all of them,
        // the lanes of a shorter channel join when m reaches their l (what they hold before that
        // is not used: the first two steps of a channel take nothing from earlier ones); bundles
        // of K channels go to the waves like single channels below
        const unsigned bundles = (static_cast<unsigned>(L - H) + K - 1u) / K;
        for (unsigned i = 0; i < bundles; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l0 = L - static_cast<int>(i * K); // >= H + 1, so l0 - (K - 1) >= 0
            ChannelPrefactors<T> pk[K], qk[K];
#pragma unroll
            for (unsigned k = 0; k < K; ++k) {
                const int lk = l0 - static_cast<int>(k);
                pk[k] = ChannelPrefactors<T>(table_F<T>() + lk * (lk + 1) / 2, lk, lane);
                qk[k] = ChannelPrefactors<T>(table_Q<T>() + lk * (lk + 1) / 2, lk, lane);
            }
            if (point >= valid) continue; // (all lanes are back at the next bundle's loads)
            const int l = l0 - static_cast<int>(side);
            const bool live = l > H;
            T* mid = row + l * l + l;
            auto prefactors = [&](int m, T& f, T& q) {
                f = pk[0][m];
                q = qk[0][m];
#pragma unroll
                for (unsigned k = 1; k < K; ++k) {
                    const T fk = pk[k][m], qk_ = qk[k][m];
                    if (side == k) {
                        f = fk;
                        q = qk_;
                    }
                }
            };
            T v1 = 0, v2 = 0;
            T c = tab[3 * l0], s = tab[3 * l0 + 1], tz = tab[3 * l0 + 2];
            for (int m = l0; m >= 1; --m) {
                const T c0 = c, s0 = s, tz0 = tz;
                c = tab[3 * m - 3];
                s = tab[3 * m - 2];
                tz = tab[3 * m - 1];
                T f, q;
                prefactors(m, f, q);
                T v0 = q * (tz0 * v1 + rxy * v2);
                if (m == l - 1) v0 = -p.z * v1;
                if (m == l) v0 = q;
                const T pq = v0 * f;
                if (live && m <= l) {
                    mid[m] = pq * c0;
                    mid[-m] = pq * s0;
                }
                v2 = v1;
                v1 = v0;
            }
            T f, q;
            prefactors(0, f, q);
            const T v0 = q * (tz * v1 + rxy * v2);
            if (live) mid[0] = v0 * f;
        }
    } else {
        const T rxy = p.x2 + p.y2;
        // channel number i = L - l goes to wave i % waves in even rounds, backwards in odd ones
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % waves;
            if ((((i / waves) & 1u) ? waves - 1u - pos : pos) != wave) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            const ChannelPrefactors<T> pk(table_F<T>() + tri, l, lane);
            const ChannelPrefactors<T> qk(table_Q<T>() + tri, l, lane);
            if (lane >= valid) continue; // (all lanes are back at the next channel's loads)
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
            // the table entries of the next m are fetched before the arithmetic of this one
            T c = tab[3 * (l - 2)], s = tab[3 * (l - 2) + 1], tz = tab[3 * (l - 2) + 2];
            for (int m = l - 2; m >= 1; --m) {
                const T c0 = c, s0 = s, tz0 = tz;
                c = tab[3 * m - 3];
                s = tab[3 * m - 2];
                tz = tab[3 * m - 1];
                const T v0 = qk[m] * (tz0 * v1 + rxy * v2);
                const T pq = v0 * pk[m];
                mid[m] = pq * c0;
                mid[-m] = pq * s0;
                v2 = v1;
                v1 = v0;
            }
            const T v0 = qk[0] * (tz * v1 + rxy * v2);
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
//
// l_max <= 6 (H = l_max): closed forms only, no channels, no tables. The same kernel then is the
// closed forms of 16 to 64 points cut in slices for the waves of a workgroup, where
// closed_form_kernel has one wave evaluate all of them and then flush alone: with rows of four
// arrays in LDS few of its single-wave workgroups fit on a CU, and each is a long chain of
// arithmetic followed by a long run of stores.
// ---------------------------------------------------------------------------
// where the eight slices of the closed forms begin: by l for H = 6 (a slice that ends with an l
// evaluates nothing of the next), in equal parts below
template <int H> __device__ constexpr int closed_slice_start(int j) {
    constexpr int NH = (H + 1) * (H + 1);
    if (H == 6) {
        constexpr int by_l[9] = {0, 9, 16, 25, 31, 36, 41, 45, 49};
        return by_l[j];
    }
    return j * NH / 8;
}

template <typename T, bool NORM, int H, int J = 0, typename Pick>
__device__ __forceinline__ void closed_form_slices(const Point<T>& p, const Rows<T>& rows, Pick mine) {
    if constexpr (J < 8) {
        constexpr int LO = closed_slice_start<H>(J), HI = closed_slice_start<H>(J + 1);
        if constexpr (HI > LO) {
            if (mine(static_cast<unsigned>(J))) closed_form_job<T, 1, NORM, H, LO, HI>(p, rows);
        }
        closed_form_slices<T, NORM, H, J + 1>(p, rows, mine);
    }
}

template <typename T, bool NORM, int H = 6, unsigned NT = kValuesMaxThreads>
__global__ __launch_bounds__(NT) void gradients_lanes_kernel(Tiling g, const T* __restrict__ xyz,
                                                                           T* __restrict__ sph,
                                                                           T* __restrict__ dsph) {
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

    Point<T> p;
    p.x = p.y = p.z = p.x2 = p.y2 = p.z2 = p.ir = 0;
    Rows<T> rows;
    rows.ny = static_cast<int>(ny);
    rows.sph = lds + lane * g.rows_elems;
    rows.dsph = lds + g.off_dsph + lane * g.off_ddsph;
    rows.ddsph = nullptr;
    T* tab = lds + g.off_pts + lane * g.off_iter; // [m][3]: c_m, s_m, 2(m+1)z
    // Who does what. The channels above the closed forms go to the waves in snake order, the
    // longest first; the eight slices of the closed forms to the waves that have no channel, or,
    // when every wave has one, to the waves from the last backwards. No wave waits for another
    // before the rows are complete: a wave with channels makes the (c_m, s_m, 2(m+1)z) tables
    // itself (a tenth of a channel's work; the waves write the same numbers to the same places
    // and each reads back what it wrote).
    const unsigned channels = H == 6 ? static_cast<unsigned>(L - H) : 0u;
    // g.sequence_waves = 2 (few points, the time of the call is that of one workgroup; the host sees
    // to it that twice the channels leave waves over): two waves share a channel, the first
    // takes the upper half of its m, the second runs the recursions bare down to the lower half.
    const unsigned parts = g.sequence_waves == 2 ? 2u : 1u;
    const unsigned channel_waves = channels * parts;
    const bool has_channel = wave < channel_waves;
    const unsigned spare = waves > channel_waves ? waves - channel_waves : 0u; // waves without a channel
    auto my_slice = [&](unsigned j) -> bool {
        return spare != 0 ? wave == channel_waves + j % spare : (waves - 1u - wave) == j % waves;
    };
    if (lane < valid) {
        p = load_point<T, NORM>(xyz + (first + lane) * 3);
        if (has_channel) {
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
        closed_form_slices<T, NORM, H>(p, rows, my_slice);
    }
    if (H == 6 && lane < valid) {
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
            if (parts == 1 ? (((i / waves) & 1u) ? waves - 1u - pos : pos) != wave : i != wave / 2u) continue;
            const int l = L - static_cast<int>(i);
            // the values of m this wave turns into entries: all, or one half of l .. 0 (m = l and
            // m = l - 1 cost less than the others, the lower half has the bare steps before it)
            const int m_top = parts == 1 || (wave & 1u) == 0 ? l : l / 2 - 1;
            const int m_bottom = parts == 1 || (wave & 1u) != 0 ? 0 : l / 2;
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
            if (m_top >= l) {
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
            if (m_top >= l - 1 && m_bottom <= l - 1) {
                // m = l - 1 (:154-198)
                const T pkm = pk[l - 1];
                auto pq = a1 * pkm;
                const T vp = pq * c0, vn = pq * s0;
                pq *= (l - 1);
                auto pdq = pkm * (l + l - 1) * b1;
                stage<T, 1, NORM>(rows, mid + l - 1, p, entry(vp, pq * c1, pq * -s1, pdq * c0));
                stage<T, 1, NORM>(rows, mid - (l - 1), p, entry(vn, pq * s1, pq * c1, pdq * s0));
            }
            for (int m = l - 2; m >= 1 && m >= m_bottom; --m) {
                // :201-390
                c0 = c1;
                s0 = s1;
                c1 = tab[3 * (m - 1)];
                s1 = tab[3 * (m - 1) + 1];
                const T tz = tab[3 * m + 2];
                const T a0 = qk[m] * (tz * a1 + rxy * a2);
                const T b0 = kb[m] * (tz * b1 + rxy * b2);
                if (m <= m_top) {
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
                }
                a2 = a1;
                a1 = a0;
                b2 = b1;
                b1 = b0;
            }
            if (m_bottom == 0) {
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
// g.sequence_waves (1, 2 or 4): the waves that share one channel, each taking a part of its m.
// ---------------------------------------------------------------------------
template <typename T, bool NORM>
__global__ __launch_bounds__(hessian_lane_threads<T>()) void hessians_lanes_kernel(Tiling g, const T* __restrict__ xyz,
                                                                            T* __restrict__ sph,
                                                                            T* __restrict__ dsph,
                                                                            T* __restrict__ ddsph) {
    constexpr int H = 1;
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
        // every wave has a channel and makes the tables for it itself (a few percent of a
        // channel's work; the waves write the same numbers to the same places and each reads back
        // what it wrote): no wave waits for another before the rows are complete
        azimuth_job<T>(p, L, c, sn, tmz);
        if (wave == waves - 1) closed_form_job<T, 2, NORM, H>(p, rows);
    }
    if (lane < valid) {
        const T rxy = p.x2 + p.y2;
        const T* cF = table_F<T>();
        const T* cQ = table_Q<T>();
        T* A = lds + g.off_jobs + (wave * tile + lane) * g.jobs_per_point;
        T* B = A + (L + 1);
        T* C = B + (L + 1);
        // The waves that share a channel each run its three recursions (a few percent of the
        // entries' work) and take a part of its m: few channels then still fill the workgroup.
        const unsigned parts = g.sequence_waves;
        const unsigned slots = waves / parts; // channels in work at a time
        const unsigned slot = wave % slots, part = wave / slots;
        for (unsigned i = 0; static_cast<int>(i) < L - H; ++i) {
            const unsigned pos = i % slots;
            if ((((i / slots) & 1u) ? slots - 1u - pos : pos) != slot) continue;
            const int l = L - static_cast<int>(i);
            const int tri = l * (l + 1) / 2;
            sequence_job<T>(l, 0, p.z, rxy, cQ, tmz, A);
            sequence_job<T>(l, 1, p.z, rxy, cQ, tmz, B);
            sequence_job<T>(l, 2, p.z, rxy, cQ, tmz, C);
            // m = l .. 0 in `parts` runs of nearly equal length, the first from the top
            const int count = l + 1;
            const int m_hi = l - static_cast<int>(part) * count / static_cast<int>(parts);
            const int m_lo = l + 1 - static_cast<int>(part + 1) * count / static_cast<int>(parts);
            for (int m = m_hi; m >= m_lo; --m) {
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

} // namespace sphx

#endif
