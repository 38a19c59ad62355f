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
// rows mirror the layout of the output arrays in HBM.
template <typename T> struct Rows {
    T* sph;
    T* dsph;
    T* ddsph;
    int ny;
};

// Normalised coordinates of one point as every job needs them.
template <typename T> struct Point {
    T x, y, z, x2, y2, z2, ir;
};

// templates.hpp:156-173 / :386-400
template <typename T, bool NORM> __device__ __forceinline__ Point<T> load_point(const T* xyz) {
    Point<T> p;
    p.x = xyz[0];
    p.y = xyz[1];
    p.z = xyz[2];
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
template <typename T, int MODE>
__device__ __forceinline__ void put(const Rows<T>& out, int k, const Entry<T>& e) {
    out.sph[k] = e.v;
    if constexpr (MODE >= 1) {
        const int ny = out.ny;
        out.dsph[k] = e.gx;
        out.dsph[ny + k] = e.gy;
        out.dsph[2 * ny + k] = e.gz;
        if constexpr (MODE == 2) {
            out.ddsph[k] = e.hxx;
            out.ddsph[ny + k] = e.hxy;
            out.ddsph[2 * ny + k] = e.hxz;
            out.ddsph[3 * ny + k] = e.hxy;
            out.ddsph[4 * ny + k] = e.hyy;
            out.ddsph[5 * ny + k] = e.hyz;
            out.ddsph[6 * ny + k] = e.hxz;
            out.ddsph[7 * ny + k] = e.hyz;
            out.ddsph[8 * ny + k] = e.hzz;
        }
    }
}

template <typename T, int MODE, bool NORM>
__device__ __forceinline__ void stage(const Rows<T>& out, int k, const Point<T>& p, Entry<T> e) {
    put<T, MODE>(out, k, finish<T, MODE, NORM>(p, e));
}

// ---- l = 0..H in closed form, one point per lane ---------------------------
//
// All (H+1)^2 values and, if asked, their gradients stay in VGPRs until they
// are staged. Second derivatives of l <= 1 vanish identically
// (macros.hpp:56-131), which is the only case MODE == 2 reaches here.
template <typename T, int MODE, bool NORM, int H>
__device__ __forceinline__ void closed_form_job(const Point<T>& p, const Rows<T>& out) {
    static_assert(MODE < 2 || H <= 1, "second derivatives in closed form stop at l = 1");
    constexpr int NH = (H + 1) * (H + 1);
    T Y[NH];
    low_values<T, H>(p.x, p.y, p.z, p.x2, p.y2, p.z2, Y);
    if constexpr (MODE == 0) {
#pragma unroll
        for (int k = 0; k < NH; ++k) {
            out.sph[k] = Y[k];
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
            stage<T, MODE, NORM>(out, k, p, e);
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
template <typename T>
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
    out[l] = v2;
    out[l - 1] = v1;
    int m = l - 2;
    if (which == 2) {
        // first step of the Q_{l-2} sequence: its start value itself (:228-231, :404-406)
        const T v0 = qk[-l - 1];
        out[m] = v0;
        v2 = v1;
        v1 = v0;
        --m;
    }
    if (m < 0) return;
    // the constants of a step do not depend on the iterates: fetch them one step ahead so that
    // the chain of dependent operations never waits for LDS
    T tz_next = tmz[m];
    T k_next = k[m];
    for (; m >= 0; --m) {
        const T tz = tz_next;
        const T km = k_next;
        const int ahead = m > 0 ? m - 1 : 0;
        tz_next = tmz[ahead];
        k_next = k[ahead];
        const T v0 = km * (tz * v1 + rxy * v2);
        out[m] = v0;
        v2 = v1;
        v1 = v0;
    }
}

// ---- the entries (l, +m) and (l, -m) of one point ---------------------------
//
// templates_core.hpp:122-152 (|m| = l), :154-198 (|m| = l - 1), :201-390
// (l - 2 >= |m| >= 1) and :392-426 (m = 0), with the Q iterates read from the
// arrays the sequence jobs left in LDS. pk is the (l, .) row of the prefactor block, c / s the
// point's azimuthal tables.
template <typename T, int MODE, bool NORM>
__device__ __forceinline__ void entry_job(int l, int m, int tri, const Point<T>& p,
                                          const T* __restrict__ pk, const T* __restrict__ c,
                                          const T* __restrict__ s, const T* __restrict__ A,
                                          [[maybe_unused]] const T* __restrict__ B,
                                          [[maybe_unused]] const T* __restrict__ C,
                                          const Rows<T>& out) {
    // tri = l(l+1)/2; pk, A, B, C already point at the (l, 0) entries of their triangular arrays
    constexpr bool GRAD = MODE >= 1;
    constexpr bool HESS = MODE == 2;
    const T x = p.x, y = p.y, z = p.z;
    const int mid = 2 * tri;
    const T zero = static_cast<T>(0.0);
    [[maybe_unused]] T x2 = 0, y2 = 0, xy = 0;
    if constexpr (HESS) {
        x2 = x * x;
        y2 = y * y;
        xy = x * y;
    }
    (void)z;

    Entry<T> neg, pos;
    neg.gx = neg.gy = neg.gz = pos.gx = pos.gy = pos.gz = zero;
    neg.hxx = neg.hxy = neg.hxz = neg.hyy = neg.hyz = neg.hzz = zero;
    pos.hxx = pos.hxy = pos.hxz = pos.hyy = pos.hyz = pos.hzz = zero;

    if (m == l) {
        // :122-152
        const T qlm_2 = A[l];
        auto pq = qlm_2 * pk[l];
        neg.v = pq * s[l];
        pos.v = pq * c[l];
        if constexpr (GRAD) {
            pq *= l;
            neg.gx = pq * s[l - 1];
            neg.gy = pos.gx = pq * c[l - 1];
            pos.gy = -neg.gx;
            if constexpr (HESS) {
                pq *= (l - 1);
                pos.hxx = pq * c[l - 2];
                neg.hxx = pq * s[l - 2];
                pos.hxy = neg.hyy = -neg.hxx;
                neg.hxy = pos.hxx;
                pos.hyy = -pos.hxx;
            }
        }
    } else if (m == l - 1) {
        // :154-198
        const T qlm_2 = A[l];
        const T qlm_1 = A[l - 1];
        auto pq = qlm_1 * pk[l - 1];
        neg.v = pq * s[l - 1];
        pos.v = pq * c[l - 1];
        if constexpr (GRAD) {
            pq *= (l - 1);
            neg.gx = pq * s[l - 2];
            neg.gy = pos.gx = pq * c[l - 2];
            pos.gy = -neg.gx;
            const T ql1m_1 = B[l - 1];
            auto pdq = pk[l - 1] * (l + l - 1) * ql1m_1;
            neg.gz = pdq * s[l - 1];
            pos.gz = pdq * c[l - 1];
            if constexpr (HESS) {
                pq *= (l - 2);
                if (l == 2) {
                    pos.hxx = 0;
                    neg.hxx = 0;
                } else {
                    pos.hxx = pq * c[l - 3];
                    neg.hxx = pq * s[l - 3];
                }
                pos.hxy = neg.hyy = -neg.hxx;
                neg.hxy = pos.hxx;
                auto temp = -pk[l - 1] * (l - 1) * qlm_2;
                pos.hxz = temp * c[l - 2];
                neg.hxz = temp * s[l - 2];
                pos.hyy = -pos.hxx;
                pos.hyz = -neg.hxz;
                neg.hyz = pos.hxz;
            }
        }
    } else if (m > 0) {
        // :201-390
        const T cm = c[m], sm = s[m], pkm = pk[m];
        const T qlm_0 = A[m];
        auto pq = qlm_0 * pkm;
        neg.v = pq * sm;
        pos.v = pq * cm;
        if constexpr (GRAD) {
            const T cm1 = c[m - 1], sm1 = s[m - 1];
            // the reference reads these after its shift: ql1m_2 is the iterate of step m + 1
            // (or the start value), ql1m_1 the iterate of step m
            const T ql1m_2 = B[m + 1];
            const T ql1m_1 = B[m];
            pq *= m;
            auto pqs = pq * sm1, pqc = pq * cm1;
            auto pdq = pkm * ql1m_2;
            auto pdqx = pdq * x;
            neg.gx = (pdqx * sm + pqs);
            pos.gx = (pdqx * cm + pqc);
            auto pdqy = pdq * y;
            neg.gy = (pdqy * sm + pqc);
            pos.gy = (pdqy * cm - pqs);
            pdq = pkm * (l + m) * ql1m_1;
            neg.gz = pdq * sm;
            pos.gz = pdq * cm;

            if constexpr (HESS) {
                // ... and these before its shift: the iterates of steps m + 2, m + 1 and m
                const T ql2m_2 = C[m + 2];
                const T ql2m_1 = C[m + 1];
                const T ql2m_0 = C[m];
                pq /= m;
                auto pql1m_1 = pkm * ql1m_2;
                auto pql2m_2 = pkm * ql2m_2;
                auto pql2m_0 = pkm * ql2m_0;
                auto pql1m_0 = pkm * ql1m_1;
                auto pql2m_1 = pkm * ql2m_1;

                T mmpqc2 = 0.0;
                T mmpqs2 = 0.0;
                if (m != 1) {
                    mmpqc2 = m * (m - 1) * pq * c[m - 2];
                    mmpqs2 = m * (m - 1) * pq * s[m - 2];
                }

                pos.hxx = pql1m_1 * cm + x2 * pql2m_2 * cm + 2 * m * x * pql1m_1 * cm1 + mmpqc2;
                neg.hxx = pql1m_1 * sm + x2 * pql2m_2 * sm + 2 * m * x * pql1m_1 * sm1 + mmpqs2;
                pos.hyy = pql1m_1 * cm + y2 * pql2m_2 * cm - 2 * m * y * pql1m_1 * sm1 - mmpqc2;
                neg.hyy = pql1m_1 * sm + y2 * pql2m_2 * sm + 2 * m * y * pql1m_1 * cm1 - mmpqs2;
                pos.hzz = (l + m) * (l + m - 1) * pql2m_0 * cm;
                neg.hzz = (l + m) * (l + m - 1) * pql2m_0 * sm;

                pos.hxy = xy * pql2m_2 * cm + y * pql1m_1 * m * cm1 - x * pql1m_1 * m * sm1 - mmpqs2;
                neg.hxy = xy * pql2m_2 * sm + y * pql1m_1 * m * sm1 + x * pql1m_1 * m * cm1 + mmpqc2;
                pos.hxz = x * (l + m) * pql2m_1 * cm + (l + m) * pql1m_0 * m * cm1;
                neg.hxz = x * (l + m) * pql2m_1 * sm + (l + m) * pql1m_0 * m * sm1;
                pos.hyz = y * (l + m) * pql2m_1 * cm - (l + m) * pql1m_0 * m * sm1;
                neg.hyz = y * (l + m) * pql2m_1 * sm + (l + m) * pql1m_0 * m * cm1;
            }
        }
    } else {
        // m = 0, :392-426
        const T qlm_0 = A[0];
        pos.v = qlm_0 * pk[0];
        if constexpr (GRAD) {
            const T ql1m_1 = B[1];
            const T ql1m_0 = B[0];
            pos.gx = pk[0] * x * ql1m_1;
            pos.gy = pk[0] * y * ql1m_1;
            pos.gz = pk[0] * l * ql1m_0;
            if constexpr (HESS) {
                const T ql2m_2 = C[2];
                const T ql2m_1 = C[1];
                const T ql2m_0 = C[0];
                auto pql1m_1 = pk[0] * ql1m_1;
                auto pql2m_2 = pk[0] * ql2m_2;
                auto pql2m_0 = pk[0] * ql2m_0;
                auto pql2m_1 = pk[0] * ql2m_1;
                pos.hxx = pql1m_1 + x2 * pql2m_2;
                pos.hyy = pql1m_1 + y2 * pql2m_2;
                pos.hzz = (l) * (l - 1) * pql2m_0;
                pos.hxy = xy * pql2m_2;
                pos.hxz = x * l * pql2m_1;
                pos.hyz = y * l * pql2m_1;
            }
        }
    }
    stage<T, MODE, NORM>(out, mid + m, p, pos);
    if (m > 0) {
        stage<T, MODE, NORM>(out, mid - m, p, neg);
    }
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
template <typename T, bool STREAMING, bool PADDED>
__device__ __forceinline__ void copy_out(const T* __restrict__ staged, T* __restrict__ dst,
                                         unsigned len, unsigned row, unsigned pad, unsigned magic,
                                         unsigned tid, unsigned nthreads) {
    using V = typename Pack<T>::type;
    constexpr unsigned W = Pack<T>::width;
    const unsigned misalign = static_cast<unsigned>(reinterpret_cast<uintptr_t>(dst) & 15u);
    unsigned head = ((16u - misalign) & 15u) / static_cast<unsigned>(sizeof(T));
    if (head > len) head = len;
    const unsigned nvec = (len - head) / W;
    V* out = reinterpret_cast<V*>(dst + head) + tid;
    if (!PADDED && head == 0) {
        // not unrolled on purpose: loads and stores alternating one by one measured 3 % faster
        // than batches of four on the closed-form kernel
        const V* in = reinterpret_cast<const V*>(staged);
        V* aligned = reinterpret_cast<V*>(dst);
        for (unsigned g = tid; g < nvec; g += nthreads) {
            emit<T, STREAMING>(in[g], aligned + g);
        }
    } else if (!PADDED) {
        const T* in = staged + head + tid * W;
#pragma unroll 4
        for (unsigned g = tid; g < nvec; g += nthreads, in += nthreads * W, out += nthreads) {
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
