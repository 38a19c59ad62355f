// Device-side building blocks of the spherical / solid harmonics evaluator for
// gfx950 (wave64, LDS-staged stores). Three jobs run inside one workgroup tile:
//
//   closed_form_job  one lane = one point, l = 0..H in registers
//                    (sphericart/include/templates.hpp:156-265 with the closed
//                    forms of macros.hpp; same split as the reference CPU
//                    classes, sphericart/src/sphericart.cpp:45-92)
//   azimuth_job      one lane = one point: c_m, s_m, 2(m+1)z into LDS
//                    (sphericart/include/templates.hpp:451-466)
//   sequence_job     one lane = one (point, l, sequence) triple: one of the downward-in-m
//                    three-term recursions of Q_l, Q_{l-1}, Q_{l-2}, iterates to LDS
//   entry_job        one lane = one (point, l, m) triple: the entries (l, +-m)
//                    with first and second derivatives from those iterates
//                    (together: sphericart/include/templates_core.hpp:35-427)
//
// plus the unit-sphere chain rule (templates.hpp:553-614) applied in registers
// right before an entry is staged, and copy_out, which streams a finished tile
// from LDS to HBM as contiguous 16-byte stores.
//
// All arithmetic keeps the reference's operation order; the library is built
// with -ffp-contract=off so that each source-level operation rounds once.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

#include "sphx_lowl.hpp"

namespace sphx {

// ---- small helpers --------------------------------------------------------

__device__ __forceinline__ float root(float v) { return sqrtf(v); }
__device__ __forceinline__ double root(double v) { return sqrt(v); }

template <typename T> struct Pack;
template <> struct Pack<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    static constexpr unsigned width = 4;
};
template <> struct Pack<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    static constexpr unsigned width = 2;
};

// Where the staged outputs of one point live in LDS. Element (component a,
// index k) of the point's gradient row is at dsph[a * ny + k], and so on; the
// rows mirror the layout of the output arrays in HBM. The rows may be of a
// narrower type than the arithmetic (float rows filled from float64 results,
// every number rounded once as it is stored).
template <typename O> struct Rows {
    O* sph;
    O* dsph;
    O* ddsph;
    int ny;
};

// Normalised coordinates of one point as every job needs them.
template <typename T> struct Point {
    T x, y, z, x2, y2, z2, ir;
};

// templates.hpp:156-173 / :386-400
template <typename T, bool NORM, typename I> __device__ __forceinline__ Point<T> load_point(const I* xyz) {
    Point<T> p;
    p.x = static_cast<T>(xyz[0]); // exact when the coordinates are stored narrower than T
    p.y = static_cast<T>(xyz[1]);
    p.z = static_cast<T>(xyz[2]);
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
    return p;
}

// One (l, m) entry on its way to LDS: value, gradient, the six distinct second
// derivatives (the reference assigns the symmetric partners the same number).
template <typename T> struct Entry {
    T v, gx, gy, gz, hxx, hxy, hxz, hyy, hyz, hzz;
};

// Chain rule for the polynomials evaluated at (x, y, z)/r.
// templates.hpp:572-613: the Hessian is corrected first, from the uncorrected
// gradient; then the gradient.
template <typename T, int MODE, bool NORM>
__device__ __forceinline__ Entry<T> finish(const Point<T>& p, Entry<T> e) {
    if constexpr (MODE >= 1 && NORM) {
        const T x = p.x, y = p.y, z = p.z, ir = p.ir;
        auto tmp = (e.gx * x + e.gy * y + e.gz * z);
        if constexpr (MODE == 2) {
            auto irsq = ir * ir;
            auto tmpx = x * e.hxx + y * e.hxy + z * e.hxz;
            auto tmpy = x * e.hxy + y * e.hyy + z * e.hyz;
            auto tmpz = x * e.hxz + y * e.hyz + z * e.hzz;
            auto tmp2 = x * x * e.hxx + y * y * e.hyy + z * z * e.hzz + 2 * x * y * e.hxy +
                        2 * x * z * e.hxz + 2 * y * z * e.hyz;
            T nxx = (-2 * x * tmpx + e.hxx + 3 * x * x * tmp - tmp - 2 * x * e.gx + x * x * tmp2) *
                    irsq;
            T nyy = (-2 * y * tmpy + e.hyy + 3 * y * y * tmp - tmp - 2 * y * e.gy + y * y * tmp2) *
                    irsq;
            T nzz = (-2 * z * tmpz + e.hzz + 3 * z * z * tmp - tmp - 2 * z * e.gz + z * z * tmp2) *
                    irsq;
            T nxy = (-x * tmpy - y * tmpx + e.hxy + 3 * x * y * tmp - x * e.gy - y * e.gx +
                     x * y * tmp2) *
                    irsq;
            T nxz = (-x * tmpz - z * tmpx + e.hxz + 3 * x * z * tmp - x * e.gz - z * e.gx +
                     x * z * tmp2) *
                    irsq;
            T nyz = (-z * tmpy - y * tmpz + e.hyz + 3 * y * z * tmp - z * e.gy - y * e.gz +
                     y * z * tmp2) *
                    irsq;
            e.hxx = nxx;
            e.hyy = nyy;
            e.hzz = nzz;
            e.hxy = nxy;
            e.hxz = nxz;
            e.hyz = nyz;
        }
        e.gx = (e.gx - x * tmp) * ir;
        e.gy = (e.gy - y * tmp) * ir;
        e.gz = (e.gz - z * tmp) * ir;
    }
    return e;
}

// Store a finished entry into the point's staged rows.
template <typename T, int MODE, typename O>
__device__ __forceinline__ void put(const Rows<O>& out, int k, const Entry<T>& e) {
    out.sph[k] = static_cast<O>(e.v);
    if constexpr (MODE >= 1) {
        const int ny = out.ny;
        out.dsph[k] = static_cast<O>(e.gx);
        out.dsph[ny + k] = static_cast<O>(e.gy);
        out.dsph[2 * ny + k] = static_cast<O>(e.gz);
        if constexpr (MODE == 2) {
            const O hxy = static_cast<O>(e.hxy), hxz = static_cast<O>(e.hxz), hyz = static_cast<O>(e.hyz);
            out.ddsph[k] = static_cast<O>(e.hxx);
            out.ddsph[ny + k] = hxy;
            out.ddsph[2 * ny + k] = hxz;
            out.ddsph[3 * ny + k] = hxy;
            out.ddsph[4 * ny + k] = static_cast<O>(e.hyy);
            out.ddsph[5 * ny + k] = hyz;
            out.ddsph[6 * ny + k] = hxz;
            out.ddsph[7 * ny + k] = hyz;
            out.ddsph[8 * ny + k] = static_cast<O>(e.hzz);
        }
    }
}

template <typename T, int MODE, bool NORM, typename O>
__device__ __forceinline__ void stage(const Rows<O>& out, int k, const Point<T>& p, Entry<T> e) {
    put<T, MODE>(out, k, finish<T, MODE, NORM>(p, e));
}

// ---- l = 0..H in closed form, one point per lane ---------------------------
//
// All (H+1)^2 values and, if asked, their gradients stay in VGPRs until they
// are staged. Second derivatives of l <= 1 vanish identically
// (macros.hpp:56-131), which is the only case MODE == 2 reaches here.
// KLO, KHI: only the entries KLO <= k < KHI are staged. The closed forms of one l use values of
// lower l but hardly any gradients of lower l, so what a slice does not stage the compiler
// drops: several waves can share the entries of a point, each evaluating little more than its
// own slice.
template <typename T, int MODE, bool NORM, int H, int KLO = 0, int KHI = (H + 1) * (H + 1), typename O = T>
__device__ __forceinline__ void closed_form_job(const Point<T>& p, const Rows<O>& out) {
    static_assert(MODE < 2 || H <= 1, "second derivatives in closed form stop at l = 1");
    constexpr int NH = (H + 1) * (H + 1);
    T Y[NH];
    low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
    if constexpr (MODE == 0) {
#pragma unroll
        for (int k = KLO; k < KHI; ++k) {
            out.sph[k] = static_cast<O>(Y[k]);
        }
    } else {
        T DX[NH], DY[NH], DZ[NH];
        low_gradients<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y, DX, DY, DZ);
        auto finished = [&](int k) {
            Entry<T> e;
            e.v = Y[k];
            e.gx = DX[k];
            e.gy = DY[k];
            e.gz = DZ[k];
            e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = static_cast<T>(0.0);
            return finish<T, MODE, NORM>(p, e);
        };
#pragma unroll
        for (int k = KLO; k < KHI; ++k) {
            put<T, MODE>(out, k, finished(k));
        }
    }
}

// Same, but the finished entries are handed back in registers so that the
// caller can stage them in several passes through a small LDS buffer.
template <typename T, int MODE, bool NORM, int H>
__device__ __forceinline__ void closed_form_entries(const Point<T>& p,
                                                    Entry<T> (&E)[(H + 1) * (H + 1)]) {
    static_assert(MODE < 2 || H <= 1, "second derivatives in closed form stop at l = 1");
    constexpr int NH = (H + 1) * (H + 1);
    T Y[NH];
    low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
    if constexpr (MODE == 0) {
#pragma unroll
        for (int k = 0; k < NH; ++k) {
            E[k].v = Y[k];
        }
    } else {
        T DX[NH], DY[NH], DZ[NH];
        low_gradients<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y, DX, DY, DZ);
#pragma unroll
        for (int k = 0; k < NH; ++k) {
            Entry<T> e;
            e.v = Y[k];
            e.gx = DX[k];
            e.gy = DY[k];
            e.gz = DZ[k];
            e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = static_cast<T>(0.0);
            E[k] = finish<T, MODE, NORM>(p, e);
        }
    }
}

// ---- c_m, s_m, 2(m+1)z for one point ---------------------------------------
// templates.hpp:451-466. The running sum for 2(m+1)z is kept as a sum: it
// rounds differently from a product.
template <typename T>
__device__ __forceinline__ void azimuth_job(const Point<T>& p, int L, T* c, T* s, T* tmz) {
    T twoz = p.z + p.z;
    T cm = 1.0, sm = 0.0, tz = twoz;
    c[0] = cm;
    s[0] = sm;
    tmz[0] = tz;
    for (int m = 1; m <= L; ++m) {
        T cn = cm * p.x - sm * p.y;
        T sn = cm * p.y + sm * p.x;
        tz = tz + twoz;
        cm = cn;
        sm = sn;
        c[m] = cm;
        s[m] = sm;
        tmz[m] = tz;
    }
}

// ---- one bare recursion of one l channel -----------------------------------
//
// For one point and one l the reference runs three three-term recursions
// downward in m side by side (templates_core.hpp:202-204, :210-212, :228-235
// with the start values of :122-123,135,150,155,167,196 and the m = 0 steps of
// :393,397,404-409):
//   which = 0:  A[m] = Q_l^m                 (its qlm_0 at step m)
//   which = 1:  B[m] = the Q_{l-1} sequence  (ql1m_0; B[l] = 0, B[l-1] = Q_{l-1}^{l-1})
//   which = 2:  C[m] = the Q_{l-2} sequence  (ql2m_0; C[l] = C[l-1] = 0, C[l-2] = Q_{l-2}^{l-2})
// They share the form v_m = k_m (2(m+1)z v_{m+1} + (x^2+y^2) v_{m+2}) and differ in
// start values and in which row of the constant table k_m comes from, so each
// is one job here, every iterate written to LDS. A recursion step is a handful
// of operations while turning an iterate into output entries costs a hundred
// or more: the iterates are computed once by a few lanes and the entries are
// then independent jobs (entry_job) for all lanes of the workgroup. Same
// operations in the same order as the reference's fused loop, hence the same
// numbers.
// STRIDE: distance in `out` between the iterates of consecutive m (1: an array of its own per
// sequence; more: the sequences of one l interleaved, `out` then points at this sequence's m = 0).
template <typename T, int STRIDE = 1>
__device__ __forceinline__ void sequence_job(int l, int which, T z, T rxy,
                                             const T* __restrict__ Q,
                                             const T* __restrict__ tmz, T* __restrict__ out) {
    const T* qk = Q + l * (l + 1) / 2;
    // row of the constant table: (l, m) for A, (l-1, m) for B, (l-2, m) for C
    const T* k = which == 0 ? qk : (which == 1 ? qk - l : qk - 2 * l + 1);
    T v2, v1;
    if (which == 0) {
        v2 = qk[l];
        v1 = -z * v2;
    } else if (which == 1) {
        v2 = 0;
        v1 = qk[-1];
    } else {
        v2 = 0.0;
        v1 = 0.0;
    }
    out[l * STRIDE] = v2;
    out[(l - 1) * STRIDE] = v1;
    int m = l - 2;
    if (which == 2) {
        // first step of the Q_{l-2} sequence: its start value itself (:228-231, :404-406)
        const T v0 = qk[-l - 1];
        out[m * STRIDE] = v0;
        v2 = v1;
        v1 = v0;
        --m;
    }
    if (m < 0) return;
    // The constants of a step (2(m+1)z and k_m) do not depend on the iterates, the steps do
    // depend on one another: a step that waited for its own constants would take one LDS round
    // trip, several times the arithmetic. So the constants are fetched DEPTH steps ahead, a
    // block of DEPTH at a time, while the block before is being worked through.
    constexpr int DEPTH = 4;
    for (int odd = (m + 1) & (DEPTH - 1); odd > 0; --odd, --m) {
        const T v0 = k[m] * (tmz[m] * v1 + rxy * v2);
        out[m * STRIDE] = v0;
        v2 = v1;
        v1 = v0;
    }
    if (m < 0) return;
    // m + 1 is a multiple of DEPTH from here on; element j of a block belongs to step base + j
    T tz[DEPTH], km[DEPTH];
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
        tz[j] = tmz[m - (DEPTH - 1) + j];
        km[j] = k[m - (DEPTH - 1) + j];
    }
    for (; m >= 0; m -= DEPTH) {
        const int base = m - (DEPTH - 1);
        const int next = base >= DEPTH ? base - DEPTH : 0; // the last block fetches, unused, from 0
        T tz_next[DEPTH], km_next[DEPTH];
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            tz_next[j] = tmz[next + j];
            km_next[j] = k[next + j];
        }
#pragma unroll
        for (int j = DEPTH - 1; j >= 0; --j) {
            const T v0 = km[j] * (tz[j] * v1 + rxy * v2);
            out[(base + j) * STRIDE] = v0;
            v2 = v1;
            v1 = v0;
        }
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) {
            tz[j] = tz_next[j];
            km[j] = km_next[j];
        }
    }
}

// ---- the entries (l, +m) and (l, -m) of one point ---------------------------
//
// templates_core.hpp:122-152 (|m| = l), :154-198 (|m| = l - 1), :201-390
// (l - 2 >= |m| >= 1) and :392-426 (m = 0), with the Q iterates read from the
// arrays the sequence jobs left in LDS. pk is the (l, .) row of the prefactor block, c / s the
// point's azimuthal tables.
//
// The reference writes the entry (l, +m) with c_m, c_{m-1}, c_{m-2} and the entry (l, -m) with
// s_m, s_{m-1}, s_{m-2} in their place; where the two formulas differ beyond that, one has
// "+ t c_{m-1}" where the other has "- t s_{m-1}" (same for m - 2). Both are written here once,
// as a function of the side: u_k stands for c_k or s_k, w_k for -s_k or c_k. Negating a factor
// negates the rounded product exactly and a + (-b) is a - b, so the numbers are the
// reference's. SPLIT == false: one job computes both sides (the common factors are shared).
// SPLIT == true: one job computes the side it is given, so that a tile with few (l, m) pairs
// still spreads over all lanes.
//
// The inputs come through `in`, addressed relative to the job's own m: in.pk() is the prefactor F_l^m,
// in.c(d) / in.s(d) are c_{m+d} / s_{m+d}, in.A(d) / in.B(d) / in.C(d) the iterates of the three recursions at
// m + d, with d a literal everywhere. A caller that holds them in arrays indexes those (EntryArrays below); a
// caller that holds them in registers answers each d with a register.
template <typename T, int MODE, bool NORM, bool SPLIT, typename In, typename O>
__device__ __forceinline__ void entry_job_from(int l, int m, int tri, int side, const Point<T>& p, const In& in,
                                               const Rows<O>& out) {
    // tri = l(l+1)/2
    constexpr bool GRAD = MODE >= 1;
    constexpr bool HESS = MODE == 2;
    const T x = p.x, y = p.y;
    const int mid = 2 * tri;
    const T zero = static_cast<T>(0.0);
    [[maybe_unused]] T x2 = 0, y2 = 0, xy = 0;
    if constexpr (HESS) {
        x2 = x * x;
        y2 = y * y;
        xy = x * y;
    }
    auto blank = [&]() {
        Entry<T> e;
        e.v = e.gx = e.gy = e.gz = zero;
        e.hxx = e.hxy = e.hxz = e.hyy = e.hyz = e.hzz = zero;
        return e;
    };
    // stage what `make(side)` returns: both sides, or the one this job was given
    auto emit_sides = [&](auto make) {
        if constexpr (SPLIT) {
            stage<T, MODE, NORM>(out, side ? mid - m : mid + m, p, make(side != 0));
        } else {
            stage<T, MODE, NORM>(out, mid + m, p, make(false));
            stage<T, MODE, NORM>(out, mid - m, p, make(true));
        }
    };

    if (m == l) {
        // :122-152
        const T qlm_2 = in.A(0);
        const T cl = in.c(0), sl = in.s(0);
        [[maybe_unused]] T cl1 = 0, sl1 = 0, cl2 = 0, sl2 = 0;
        if constexpr (GRAD) {
            cl1 = in.c(-1);
            sl1 = in.s(-1);
        }
        if constexpr (HESS) {
            cl2 = in.c(-2);
            sl2 = in.s(-2);
        }
        emit_sides([&](bool minus) {
            Entry<T> e = blank();
            auto pq = qlm_2 * in.pk();
            e.v = pq * (minus ? sl : cl);
            if constexpr (GRAD) {
                pq *= l;
                e.gx = pq * (minus ? sl1 : cl1);
                e.gy = pq * (minus ? cl1 : -sl1);
                if constexpr (HESS) {
                    pq *= (l - 1);
                    e.hxx = pq * (minus ? sl2 : cl2);
                    e.hxy = pq * (minus ? cl2 : -sl2);
                    e.hyy = -e.hxx;
                }
            }
            return e;
        });
    } else if (m == l - 1) {
        // :154-198
        [[maybe_unused]] const T qlm_2 = in.A(1);
        const T qlm_1 = in.A(0);
        const T pkm = in.pk();
        const T cm = in.c(0), sm = in.s(0);
        [[maybe_unused]] T cm1 = 0, sm1 = 0, cm2 = 0, sm2 = 0, ql1m_1 = 0;
        if constexpr (GRAD) {
            cm1 = in.c(-1);
            sm1 = in.s(-1);
            ql1m_1 = in.B(0);
        }
        if constexpr (HESS) {
            if (l != 2) {
                cm2 = in.c(-2);
                sm2 = in.s(-2);
            }
        }
        emit_sides([&](bool minus) {
            Entry<T> e = blank();
            auto pq = qlm_1 * pkm;
            e.v = pq * (minus ? sm : cm);
            if constexpr (GRAD) {
                pq *= (l - 1);
                e.gx = pq * (minus ? sm1 : cm1);
                e.gy = pq * (minus ? cm1 : -sm1);
                auto pdq = pkm * (l + l - 1) * ql1m_1;
                e.gz = pdq * (minus ? sm : cm);
                if constexpr (HESS) {
                    pq *= (l - 2);
                    if (l == 2) {
                        // the reference sets xx to zero and derives the rest from it by negation
                        e.hxx = zero;
                        e.hxy = minus ? zero : -zero;
                    } else {
                        e.hxx = pq * (minus ? sm2 : cm2);
                        e.hxy = pq * (minus ? cm2 : -sm2);
                    }
                    e.hyy = -e.hxx;
                    auto temp = -pkm * (l - 1) * qlm_2;
                    e.hxz = temp * (minus ? sm1 : cm1);
                    e.hyz = temp * (minus ? cm1 : -sm1);
                }
            }
            return e;
        });
    } else if (m > 0) {
        // :201-390
        const T cm = in.c(0), sm = in.s(0), pkm = in.pk();
        const T qlm_0 = in.A(0);
        [[maybe_unused]] T cm1 = 0, sm1 = 0, cm2 = 0, sm2 = 0, ql1m_2 = 0, ql1m_1 = 0;
        [[maybe_unused]] T ql2m_2 = 0, ql2m_1 = 0, ql2m_0 = 0;
        if constexpr (GRAD) {
            cm1 = in.c(-1);
            sm1 = in.s(-1);
            // the reference reads these after its shift: ql1m_2 is the iterate of step m + 1
            // (or the start value), ql1m_1 the iterate of step m
            ql1m_2 = in.B(1);
            ql1m_1 = in.B(0);
        }
        if constexpr (HESS) {
            // ... and these before its shift: the iterates of steps m + 2, m + 1 and m
            ql2m_2 = in.C(2);
            ql2m_1 = in.C(1);
            ql2m_0 = in.C(0);
            if (m != 1) {
                cm2 = in.c(-2);
                sm2 = in.s(-2);
            }
        }
        emit_sides([&](bool minus) {
            Entry<T> e = blank();
            const T u = minus ? sm : cm;
            auto pq = qlm_0 * pkm;
            e.v = pq * u;
            if constexpr (GRAD) {
                const T u1 = minus ? sm1 : cm1;
                const T w1 = minus ? cm1 : -sm1;
                pq *= m;
                auto pdq = pkm * ql1m_2;
                auto pdqx = pdq * x;
                e.gx = (pdqx * u + pq * u1);
                auto pdqy = pdq * y;
                e.gy = (pdqy * u + pq * w1);
                pdq = pkm * (l + m) * ql1m_1;
                e.gz = pdq * u;

                if constexpr (HESS) {
                    pq /= m;
                    auto pql1m_1 = pkm * ql1m_2;
                    auto pql2m_2 = pkm * ql2m_2;
                    auto pql2m_0 = pkm * ql2m_0;
                    auto pql1m_0 = pkm * ql1m_1;
                    auto pql2m_1 = pkm * ql2m_1;

                    // m (m-1) pq u_{m-2} and m (m-1) pq w_{m-2}
                    T mmpqu2 = 0.0;
                    T mmpqw2 = 0.0;
                    if (m != 1) {
                        mmpqu2 = m * (m - 1) * pq * (minus ? sm2 : cm2);
                        mmpqw2 = m * (m - 1) * pq * (minus ? cm2 : -sm2);
                    }

                    e.hxx = pql1m_1 * u + x2 * pql2m_2 * u + 2 * m * x * pql1m_1 * u1 + mmpqu2;
                    e.hyy = pql1m_1 * u + y2 * pql2m_2 * u + 2 * m * y * pql1m_1 * w1 - mmpqu2;
                    e.hzz = (l + m) * (l + m - 1) * pql2m_0 * u;
                    e.hxy = xy * pql2m_2 * u + y * pql1m_1 * m * u1 + x * pql1m_1 * m * w1 + mmpqw2;
                    e.hxz = x * (l + m) * pql2m_1 * u + (l + m) * pql1m_0 * m * u1;
                    e.hyz = y * (l + m) * pql2m_1 * u + (l + m) * pql1m_0 * m * w1;
                }
            }
            return e;
        });
    } else {
        // m = 0, :392-426
        Entry<T> pos = blank();
        const T qlm_0 = in.A(0);
        const T pk0 = in.pk();
        pos.v = qlm_0 * pk0;
        if constexpr (GRAD) {
            const T ql1m_1 = in.B(1);
            const T ql1m_0 = in.B(0);
            pos.gx = pk0 * x * ql1m_1;
            pos.gy = pk0 * y * ql1m_1;
            pos.gz = pk0 * l * ql1m_0;
            if constexpr (HESS) {
                const T ql2m_2 = in.C(2);
                const T ql2m_1 = in.C(1);
                const T ql2m_0 = in.C(0);
                auto pql1m_1 = pk0 * ql1m_1;
                auto pql2m_2 = pk0 * ql2m_2;
                auto pql2m_0 = pk0 * ql2m_0;
                auto pql2m_1 = pk0 * ql2m_1;
                pos.hxx = pql1m_1 + x2 * pql2m_2;
                pos.hyy = pql1m_1 + y2 * pql2m_2;
                pos.hzz = (l) * (l - 1) * pql2m_0;
                pos.hxy = xy * pql2m_2;
                pos.hxz = x * l * pql2m_1;
                pos.hyz = y * l * pql2m_1;
            }
        }
        stage<T, MODE, NORM>(out, mid, p, pos);
    }
}

// The inputs of entry_job_from in arrays: pk, A, B, C point at the (l, 0) entries of their triangular
// arrays, c / s at the point's azimuthal tables.
template <typename T> struct EntryArrays {
    int m;
    const T* __restrict__ pk_;
    const T* __restrict__ c_;
    const T* __restrict__ s_;
    const T* __restrict__ A_;
    const T* __restrict__ B_;
    const T* __restrict__ C_;
    __device__ __forceinline__ T pk() const { return pk_[m]; }
    __device__ __forceinline__ T c(int d) const { return c_[m + d]; }
    __device__ __forceinline__ T s(int d) const { return s_[m + d]; }
    __device__ __forceinline__ T A(int d) const { return A_[m + d]; }
    __device__ __forceinline__ T B(int d) const { return B_[m + d]; }
    __device__ __forceinline__ T C(int d) const { return C_[m + d]; }
};

template <typename T, int MODE, bool NORM, bool SPLIT, typename O>
__device__ __forceinline__ void entry_job(int l, int m, int tri, int side, const Point<T>& p,
                                          const T* __restrict__ pk, const T* __restrict__ c,
                                          const T* __restrict__ s, const T* __restrict__ A,
                                          const T* __restrict__ B, const T* __restrict__ C,
                                          const Rows<O>& out) {
    const EntryArrays<T> in{m, pk, c, s, A, B, C};
    entry_job_from<T, MODE, NORM, SPLIT>(l, m, tri, side, p, in, out);
}

// ---- LDS -> HBM ------------------------------------------------------------
//
// A tile of consecutive points is one contiguous run of `len` elements in an
// output array; in LDS the same run is stored point after point with `pad`
// spare elements after every `row` elements (row = what one point contributes;
// the pad keeps the per-point stride odd so that lanes staging the same entry
// of different points hit different banks). `magic` = ceil(2^32 / row) turns the
// division by `row` into a multiply-high; it is exact here because an LDS tile
// holds fewer than 2^16 elements.
template <typename T>
__device__ __forceinline__ unsigned staged_index(unsigned g, unsigned row, unsigned pad,
                                                 unsigned magic) {
    return g + pad * __umulhi(g, magic);
}

template <typename T, bool STREAMING, typename V>
__device__ __forceinline__ void emit(V v, V* dst) {
    if constexpr (STREAMING) {
        __builtin_nontemporal_store(v, dst);
    } else {
        *dst = v;
    }
}

// Copy `len` staged elements to dst[0 .. len). Whatever the alignment of dst, the bulk goes out
// as 16-byte stores at 16-byte aligned addresses, consecutive lanes to consecutive addresses;
// at most three (float) or one (double) leading and trailing elements are stored one by one.
// PADDED: the staged run has `pad` spare elements after every `row` elements (see staged_index).
// LINES: the 16-byte stores start at a 128-byte line of dst instead of at the first 16-byte
// boundary, so that every store instruction of a wave (64 x 16 bytes) covers eight whole lines
// and none is written in two parts by two instructions; up to 31 (float) or 15 (double)
// leading elements are then stored one by one. Needs nthreads >= 34.
template <typename T, bool STREAMING, bool PADDED, int UNROLL = 1, bool LINES = false>
__device__ __forceinline__ void copy_out(const T* __restrict__ staged, T* __restrict__ dst,
                                         unsigned len, unsigned row, unsigned pad, unsigned magic,
                                         unsigned tid, unsigned nthreads) {
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    constexpr unsigned ALIGN = LINES ? 128u : 16u;
    const unsigned misalign = static_cast<unsigned>(reinterpret_cast<uintptr_t>(dst) & (ALIGN - 1u));
    unsigned head = ((ALIGN - misalign) & (ALIGN - 1u)) / static_cast<unsigned>(sizeof(T));
    if (head > len) head = len;
    const unsigned nvec = (len - head) / W;
    V* out = reinterpret_cast<V*>(dst + head) + tid;
    if (!PADDED && head == 0) {
        // UNROLL == 1 where many waves share the copy: loads and stores alternating one by one
        // measured 3 % faster than batches of four on the closed-form kernel. A lone flushing
        // wave needs several loads in flight to keep its stores coming.
        const V* in = reinterpret_cast<const V*>(staged);
        V* aligned = reinterpret_cast<V*>(dst);
        unsigned g = tid;
        if constexpr (UNROLL > 1) {
            for (; g + (UNROLL - 1) * nthreads < nvec; g += UNROLL * nthreads) {
                V v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) v[u] = in[g + u * nthreads];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) emit<T, STREAMING>(v[u], aligned + g + u * nthreads);
            }
        }
        for (; g < nvec; g += nthreads) {
            emit<T, STREAMING>(in[g], aligned + g);
        }
    } else if (!PADDED && (reinterpret_cast<uintptr_t>(staged + head) & 15u) == 0) {
        // staged data and destination at the same position within 16 bytes: vectors on both sides
        const V* in = reinterpret_cast<const V*>(staged + head);
        unsigned g = tid;
        if constexpr (UNROLL > 1) {
            for (; g + (UNROLL - 1) * nthreads < nvec; g += UNROLL * nthreads) {
                V v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) v[u] = in[g + u * nthreads];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) emit<T, STREAMING>(v[u], out - tid + g + u * nthreads);
            }
        }
        for (; g < nvec; g += nthreads) {
            emit<T, STREAMING>(in[g], out - tid + g);
        }
    } else if (!PADDED) {
        // staged data and destination differ in their position within 16 bytes: the LDS side
        // is read element by element
        const T* in = staged + head + tid * W;
        unsigned g = tid;
        if constexpr (UNROLL > 1) {
            for (; g + (UNROLL - 1) * nthreads < nvec;
                 g += UNROLL * nthreads, in += UNROLL * nthreads * W, out += UNROLL * nthreads) {
                V v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
                    for (unsigned e = 0; e < W; ++e) v[u][e] = in[u * nthreads * W + e];
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) emit<T, STREAMING>(v[u], out + u * nthreads);
            }
        }
        for (; g < nvec; g += nthreads, in += nthreads * W, out += nthreads) {
            V v;
#pragma unroll
            for (unsigned e = 0; e < W; ++e) {
                v[e] = in[e];
            }
            emit<T, STREAMING>(v, out);
        }
    } else {
#pragma unroll 2
        for (unsigned g = tid; g < nvec; g += nthreads, out += nthreads) {
            V v;
#pragma unroll
            for (unsigned e = 0; e < W; ++e) {
                v[e] = staged[staged_index<T>(head + g * W + e, row, pad, magic)];
            }
            emit<T, STREAMING>(v, out);
        }
    }
    // leading and trailing elements
    const unsigned tail_first = head + nvec * W;
    const unsigned loose = head + (len - tail_first);
    if (tid < loose) {
        const unsigned at = tid < head ? tid : tail_first + (tid - head);
        emit<T, STREAMING>(staged[PADDED ? staged_index<T>(at, row, pad, magic) : at], dst + at);
    }
}

// The first NY entries of `count` points' component rows, staged as [count][MULT * NY + pad],
// to rows that are `ny` apart in HBM (4- or 8-byte stores, consecutive lanes to consecutive
// entries).
template <typename T, bool STREAMING, unsigned NY, unsigned MULT>
__device__ __forceinline__ void copy_prefixes(const T* staged, T* dst, unsigned count, unsigned ny,
                                              unsigned pad, unsigned tid, unsigned nthreads) {
    const unsigned total = count * MULT * NY;
    for (unsigned g = tid; g < total; g += nthreads) {
        const unsigned row = g / NY;
        const unsigned k = g - row * NY;
        const unsigned s = row / MULT;
        emit<T, STREAMING>(staged[g + pad * s], dst + static_cast<unsigned long long>(row) * ny + k);
    }
}

} // namespace sphx
