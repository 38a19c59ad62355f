// TEST INFRASTRUCTURE ONLY -- never linked into, loaded by or called from the
// shipped library. Only the test-suite, the smoke check and the CPU-baseline
// leg of the benchmark may use it, and only as the checker.
//
// CPU restatement (C++17, optional OpenMP) of the reference's host evaluator of
// real spherical harmonics Y_l^m(x/r) and solid harmonics r^l Y_l^m in
// Cartesian coordinates with first and second derivatives. Every floating-point
// operation is performed in the same order and association as the reference so
// that, compiled without FMA contraction, the results are bit-identical to the
// reference compiled the same way. Each function cites what it follows
// (paths relative to the reference checkout):
//
//   prefactors()          sphericart/include/templates.hpp:54-97
//   low_values()          sphericart/include/macros.hpp:51,76-79,133-141,161-172,
//                         201-220,259-284,344-377
//   low_gradients()       sphericart/include/macros.hpp:53-54,81-90,143-159,174-199,
//                         222-257,286-342,379-464
//   channel()             sphericart/include/templates_core.hpp:35-427
//   unit_sphere_fixup()   sphericart/include/templates.hpp:214-265,553-614
//   one_sample()          sphericart/include/templates.hpp:99-267,333-615
//   hardcoded_limit()     sphericart/src/sphericart.cpp:45-92,428-475
//   many_samples()        sphericart/include/templates.hpp:269-331,617-710
//   backward()            sphericart/src/sphericart_impl.cu:650-684 (the sum it forms; the
//                         reference adds in sub-warp order, this loop in index order)
//   backward_second()     sphericart-torch/python/sphericart/torch/register.py:106-110
//
// Pinned by (tests/test_oracle_*.py): closed-form prefactors, scipy's
// sph_harm_y up to l = 20, the Unsold sum rule, finite differences, Euler
// homogeneity, harmonicity and symmetry of the Hessian, the +-z axis values,
// the hardcoded-vs-recursion route check, bit-for-bit comparison with the
// compiled reference (oracle/_ref) where that is built, and the committed
// golden vectors written by the compiled reference. backward() and
// backward_second() are dot products: pinned against numpy's einsum in extended
// precision (tests/test_oracle_backward.py).

#include <cmath>
#include <cstddef>
#include <cstdint>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

#define K(v) static_cast<T>(v)

// ---------------------------------------------------------------------------
// F_l^m and the constants of the downward-in-m Q_l^m recursion.
// templates.hpp:54-97. Layout: two triangular blocks of (L+1)(L+2)/2 entries,
// entry (l, m) of a block at l(l+1)/2 + m.
// ---------------------------------------------------------------------------
template <typename T> void prefactors(int L, T* out) {
    const T pi = static_cast<T>(3.141592653589793238462643383279502884L);
    const T rsqrt2 = static_cast<T>(0.707106781186547524400844362104849039L);
    int at = 0;
    for (int l = 0; l <= L; ++l) {
        T run = (2 * l + 1) / (2 * pi);
        out[at] = std::sqrt(run) * rsqrt2;
        for (int m = 1; m <= l; ++m) {
            run *= static_cast<T>(1.0) / (l * (l + 1) + m * (1 - m));
            out[at + m] = (m % 2 == 0) ? std::sqrt(run) : -std::sqrt(run);
        }
        at += l + 1;
    }
    out[at] = 1;
    at += 1;
    for (int l = 1; l <= L; ++l) {
        out[at + l] = -(2 * l - 1) * out[at - 1];
        for (int m = l - 1; m >= 0; --m) {
            out[at + m] = static_cast<T>(-1.0) / ((l + m + 1) * (l - m));
        }
        at += l + 1;
    }
}

// ---------------------------------------------------------------------------
// Closed-form polynomials, l = 0..H (H <= 6). Y is indexed by l(l+1)+m.
// Higher l reuse lower-l entries, so the order of evaluation is fixed.
// macros.hpp:51-377.
// ---------------------------------------------------------------------------
template <typename T> void low_values(int H, T x, T y, T z, T x2, T y2, T z2, T* Y) {
    Y[0] = K(0.282094791773878);
    if (H < 1) return;

    Y[1] = K(0.48860251190292) * y;
    Y[2] = K(0.48860251190292) * z;
    Y[3] = K(0.48860251190292) * x;
    if (H < 2) return;

    {
        T t = K(2.23606797749979) * x;
        Y[4] = t * Y[1];
        Y[7] = t * Y[2];
        Y[5] = K(2.23606797749979) * z * Y[1];
        Y[6] = -K(0.315391565252520) * (x2 + y2 - 2 * z2);
        Y[8] = K(0.54627421529604) * (x2 - y2);
    }
    if (H < 3) return;

    {
        Y[9] = -K(0.59004358992664) * y * (y2 - 3 * x2);
        Y[10] = K(2.64575131106459) * z * Y[4];
        T t = -K(0.457045799464466) * (x2 + y2 - 4 * z2);
        Y[11] = y * t;
        Y[13] = x * t;
        Y[12] = -K(1.49270533036046) * z * (z2 - K(2.37799637856361) * Y[6]);
        Y[14] = K(1.44530572132028) * z * (x2 - y2);
        Y[15] = K(0.59004358992664) * x * (x2 - 3 * y2);
    }
    if (H < 4) return;

    {
        Y[16] = K(4.194391357527674) * Y[4] * Y[8];
        Y[17] = 3 * z * Y[9];
        T t = -K(0.866025403784439) * (x2 + y2 - 6 * z2);
        Y[18] = t * Y[4];
        Y[22] = t * Y[8];
        Y[20] = -K(0.69436507482941) *
                (y * Y[11] - K(1.6329931618554521) * z * Y[12] + x * Y[13]);
        t = -K(1.224744871391589) * (z2 - K(4.755992757127213) * Y[6]);
        Y[19] = Y[5] * t;
        Y[21] = Y[7] * t;
        Y[23] = 3 * z * Y[15];
        Y[24] = -K(1.060660171779821) * (y * Y[9] - x * Y[15]);
    }
    if (H < 5) return;

    {
        Y[25] = K(13.12764113680340) * y *
                (y2 * (x2 - K(0.2) * y2) + K(0.3994658435740642) * Y[24]);
        T t = K(3.316624790355400) * z;
        Y[26] = t * Y[16];
        Y[34] = t * Y[24];
        t = K(4.974937185533100) * (z2 + K(0.5284436396808015) * Y[6]);
        Y[27] = t * Y[9];
        Y[33] = t * Y[15];
        t = K(5.257947827012948) * Y[6];
        Y[28] = t * Y[10];
        Y[32] = t * Y[14];
        t = K(0.6324555320336759) * z;
        Y[29] = K(1.427248064296125) * (y * Y[20] + t * Y[19]);
        Y[31] = K(1.427248064296125) * (x * Y[20] + t * Y[21]);
        Y[30] = K(1.403403869441083) *
                (K(3.540173863740353) * Y[6] * Y[12] - z * z2 * z2);
        Y[35] = -K(1.048808848170152) * (y * Y[16] - x * Y[24]);
    }
    if (H < 6) return;

    {
        Y[36] = K(3.924637560539857) * Y[9] * Y[15];
        T t = K(3.605551275463989) * z;
        Y[37] = t * Y[25];
        Y[47] = t * Y[35];
        t = K(6.4498061986388) * (z2 + K(0.396332729760601) * Y[6]);
        Y[38] = t * Y[16];
        Y[46] = t * Y[24];
        t = K(1.04083299973307) * (z2 + K(4.75599275712721) * Y[6]);
        Y[39] = t * Y[17];
        Y[45] = t * Y[23];
        Y[40] = K(2.033805211017918) * (K(0.3779644730092272) * z * Y[28] + x * Y[29]);
        t = -K(6.399218702310463) * (z2 * z2 - K(4.188790204786391) * Y[6] * Y[6]);
        Y[41] = t * Y[5];
        Y[43] = t * Y[7];
        Y[42] = -K(1.087114613009218) *
                (K(0.645497224367903) * y * Y[29] - z * Y[30] + K(0.645497224367903) * x * Y[31]);
        Y[44] = -K(0.9414688716912718) *
                (y * Y[27] - K(1.63299316185545) * z * Y[32] + x * Y[33]);
        Y[48] = -K(1.040832999733066) * (y * Y[25] - x * Y[35]);
    }
}

// ---------------------------------------------------------------------------
// Closed-form first derivatives, l = 0..H, written in terms of the values and
// of derivatives assigned earlier in the same l. macros.hpp:53-464.
// ---------------------------------------------------------------------------
template <typename T>
void low_gradients(int H, T x, T y, T z, T x2, T y2, T z2, const T* Y, T* DX, T* DY, T* DZ) {
    DX[0] = DY[0] = DZ[0] = K(0.0);
    if (H < 1) return;

    DX[1] = K(0.0);
    DX[2] = K(0.0);
    DX[3] = K(0.48860251190292);
    DY[1] = K(0.48860251190292);
    DY[2] = K(0.0);
    DY[3] = K(0.0);
    DZ[1] = K(0.0);
    DZ[2] = K(0.48860251190292);
    DZ[3] = K(0.0);
    if (H < 2) return;

    DX[4] = K(2.23606797749979) * Y[1];
    DX[5] = K(0.0);
    DX[6] = -K(1.29099444873581) * Y[3];
    DX[7] = K(2.23606797749979) * Y[2];
    DX[8] = K(2.23606797749979) * Y[3];

    DY[4] = -K(1.73205080756888) * DX[6];
    DY[5] = DX[7];
    DY[6] = -K(0.577350269189626) * DX[4];
    DY[7] = K(0.0);
    DY[8] = -DX[4];

    DZ[4] = DZ[8] = K(0.0);
    DZ[5] = DX[4];
    DZ[6] = K(1.15470053837925) * DX[7];
    DZ[7] = DY[4];
    if (H < 3) return;

    DX[9] = K(3.24037034920393) * Y[4];
    DX[10] = K(2.64575131106459) * Y[5];
    DX[11] = -K(0.83666002653408) * Y[4];
    DX[12] = -K(2.04939015319192) * Y[7];
    DX[13] = K(0.91409159892893) * (y2 - z2 + K(4.75599275712721) * Y[6]);
    DX[14] = K(2.64575131106459) * Y[7];
    DX[15] = K(3.24037034920393) * Y[8];

    DY[9] = DX[15];
    DY[10] = DX[14];
    DY[11] = -K(0.91409159892893) * (y2 - z2 - K(1.58533091904240) * Y[6]);
    DY[12] = -K(2.04939015319192) * Y[5];
    DY[13] = -K(0.83666002653408) * Y[4];
    DY[14] = -DX[10];
    DY[15] = -DX[9];

    DZ[9] = K(0.0);
    DZ[10] = K(2.64575131106459) * Y[4];
    DZ[11] = K(3.34664010613630) * Y[5];
    DZ[12] = K(3.54964786985977) * Y[6];
    DZ[13] = K(3.34664010613630) * Y[7];
    DZ[14] = K(2.64575131106459) * Y[8];
    DZ[15] = K(0.0);
    if (H < 4) return;

    DX[16] = K(4.242640687119285) * Y[9];
    DX[17] = K(3.674234614174767) * Y[10];
    DX[18] = K(1.892349391515120) * y * (y2 + K(4.755992757127213) * Y[6]);
    DX[19] = -K(1.388730149658827) * Y[10];
    DX[20] = -K(2.777460299317654) * Y[13];
    DX[21] = -K(1.338093087114578) *
             (z * z2 - K(2.745873698591307) * y * Y[5] - K(4.019547514144073) * Y[12]);
    DX[22] = -K(1.892349391515120) * x * (x2 - 3 * z2);
    DX[23] = K(3.674234614174767) * Y[14];
    DX[24] = K(4.242640687119285) * Y[15];

    DY[16] = DX[24];
    DY[17] = DX[23];
    DY[18] = -K(1.892349391515120) * x * (y2 - 2 * z2 - K(1.585330919042404) * Y[6]);
    DY[19] = -K(1.338093087114578) * (z * (3 * y2 - z2) - K(1.339849171381358) * Y[12]);
    DY[20] = -K(2.777460299317654) * Y[11];
    DY[21] = DX[19];
    DY[22] = K(1.892349391515120) * y * (y2 - 3 * z2);
    DY[23] = -DX[17];
    DY[24] = -DX[16];

    DZ[16] = K(0.0);
    DZ[17] = 3 * Y[9];
    DZ[18] = K(3.927922024247863) * Y[10];
    DZ[19] = K(4.391550328268399) * Y[11];
    DZ[20] = K(4.535573676110727) * Y[12];
    DZ[21] = K(4.391550328268399) * Y[13];
    DZ[22] = K(3.927922024247863) * Y[14];
    DZ[23] = 3 * Y[15];
    DZ[24] = K(0.0);
    if (H < 5) return;

    DX[25] = K(5.244044240850758) * Y[16];
    DX[26] = K(4.690415759823430) * Y[17];
    DX[27] = K(3.582364210034113) * (y2 * Y[4] + K(3.58568582800318) * x * Y[11]);
    DX[28] = -K(8.774964387392122) * ((y2 - z2) * Y[5] + K(0.3086066999241838) * Y[17]);
    DX[29] = -K(1.914854215512676) * Y[18];
    DX[30] = -K(3.496029493900505) * Y[21];
    DX[31] = -K(8.616843969807043) *
             (K(0.2102610435016800) * z2 * z2 + K(1.056887279361603) * Y[5] * Y[5] +
              (y2 - z2) * Y[6] + K(0.555555555555556) * Y[22]);
    DX[32] = -K(8.774964387392122) * (x2 - z2) * Y[7];
    DX[33] = -K(5.170697352496190) *
             (K(0.106904496764970) * z * DX[23] - K(0.320713490294909) * y * Y[9] - Y[22]);
    DX[34] = K(4.690415759823430) * Y[23];
    DX[35] = K(5.24404424085076) * Y[24];

    DY[25] = DX[35];
    DY[26] = DX[34];
    DY[27] = -K(3.102418411497714) *
             (K(0.534522483824849) * y * Y[9] - K(0.654653670707977) * z * Y[14] - Y[22]);
    DY[28] = -K(8.77496438739212) * (y2 - K(1.585330919042404) * Y[6]) * Y[7];
    DY[29] = K(0.7237468644557459) *
             (y * (K(2.12132034355964) * Y[9] - K(8.21583836257749) * Y[11]) +
              K(6.70820393249937) * z * Y[12] + Y[24]);
    DY[30] = -K(3.496029493900505) * Y[19];
    DY[31] = DX[29];
    DY[32] = K(8.77496438739212) * (y2 - z2) * Y[5];
    DY[33] = K(3.582364210034113) * Y[4] * (y2 - 5 * z2 - K(1.585330919042404) * Y[6]);
    DY[34] = -DX[26];
    DY[35] = -DX[25];

    DZ[25] = K(0.0);
    DZ[26] = K(3.316624790355400) * Y[16];
    DZ[27] = K(4.422166387140533) * Y[17];
    DZ[28] = K(5.066228051190221) * Y[18];
    DZ[29] = K(5.416025603090640) * Y[19];
    DZ[30] = K(5.527707983925666) * Y[20];
    DZ[31] = K(5.416025603090640) * Y[21];
    DZ[32] = K(5.066228051190221) * Y[22];
    DZ[33] = K(4.422166387140533) * Y[23];
    DZ[34] = K(3.316624790355400) * Y[24];
    DZ[35] = K(0.0);
    if (H < 6) return;

    DX[36] = K(6.244997998398398) * Y[25];
    DY[48] = -DX[36];
    DX[37] = K(5.700877125495690) * Y[26];
    DY[47] = -DX[37];
    DX[38] = -K(8.07303841165959) * y *
             (y2 * y2 - K(4.188790204786391) * Y[5] * Y[5] - K(2.642218198404007) * Y[22]);
    DX[39] = -K(15.29705854077835) * ((y2 - z2) * Y[10] + K(0.2611164839335468) * Y[26]);
    DX[40] = K(32.08092506951781) *
             (Y[5] * (K(0.577350269189626) * y * Y[5] - z * Y[6]) +
              K(0.364182810197360) * y * y2 * Y[6] + K(0.3169804496925759) * Y[29]);
    DX[41] = -K(2.430862174021989) * Y[28];
    DY[43] = DX[41];
    DX[42] = -K(4.210376791603422) * Y[31];
    DY[42] = -K(4.210376791603422) * Y[29];
    DX[43] = K(4.660970900149851) *
             (z2 * z * (K(1.666666666666667) * y2 + z2 - K(2.642218198404007) * Y[6]) +
              K(1.245553603643984) * y * Y[19] + K(1.781383145961857) * Y[30]);
    DX[44] = K(14.73928415223878) *
             (x * (y2 - z2) * (2 * x2 - z2 - y2) + K(0.2856568031469765) * Y[35]);
    DX[45] = K(3.122498999199199) *
             (y * Y[17] - K(1.224744871391589) * z2 * Y[14] + +K(1.846372364689991) * Y[32]);
    {
        T t = K(1.612451549659710) * (y * Y[16] - K(1.4142135623730950) * z * Y[23]);
        DX[46] = t + K(6.18796485857095) * Y[33];
        DY[38] = -t + K(4.125309905713972) * Y[33];
    }
    DX[47] = K(5.700877125495690) * Y[34];
    DX[48] = K(6.244997998398398) * Y[35];
    DY[36] = DX[48];
    DY[37] = DX[47];
    DY[39] = -K(3.122498999199199) *
             (-K(1.22474487139159) * z2 * Y[14] + y * Y[17] - K(1.10782341881399) * Y[32]);
    DY[40] = K(11.68332144554792) *
             (x * (-K(1.585330919042404) * Y[5] * Y[5] + (z2 - y2) * Y[6]) +
              K(0.1740776559556978) * Y[31]);
    DY[41] = -K(6.99145635022478) * z *
             (z2 * z2 + (K(5.28443639680801) * y2 - K(4.188790204786391) * Y[6]) * Y[6]);
    DY[44] = K(13.49073756323204) *
             (y2 * z * Y[5] +
              (-K(0.14940357616680) * x2 + K(0.44821072850040) * y2 - K(0.59761430466720) * z2) *
                  Y[11]);
    DY[45] = K(7.648529270389177) * (y2 - z2 - K(1.58533091904240) * Y[6]) * Y[10];
    DY[46] = K(11.40175425099138) *
             (K(0.2360174359706574) * y2 * y2 * y + (y2 - 3 * z2) * Y[9] +
              K(0.1348399724926484) * Y[25]);

    DZ[36] = K(0.0);
    DZ[37] = K(3.605551275463989) * Y[25];
    DZ[38] = K(4.861724348043977) * Y[26];
    DZ[39] = K(5.64881323014763) * Y[27];
    DZ[40] = K(6.14964891828646) * Y[28];
    DZ[41] = K(6.43145678393600) * Y[29];
    DZ[42] = K(6.52268767805531) * Y[30];
    DZ[43] = K(6.43145678393600) * Y[31];
    DZ[44] = K(6.14964891828646) * Y[32];
    DZ[45] = K(5.64881323014763) * Y[33];
    DZ[46] = K(4.861724348043977) * Y[34];
    DZ[47] = K(3.605551275463989) * Y[35];
    DZ[48] = K(0.0);
}

// Second derivatives of the nine components: xx xy xz yx yy yz zx zy zz.
enum { XX = 0, XY, XZ, YX, YY, YZ, ZX, ZY, ZZ };

// ---------------------------------------------------------------------------
// One l channel through the downward-in-m Q_l^m recursion.
// templates_core.hpp:35-427. All output pointers address the m = 0 entry of
// the channel; pk / qk address the (l, 0) entries of the two prefactor blocks,
// so qk[m - l] is the (l-1, m) constant and qk[m - 2l + 1] the (l-2, m) one.
// c, s, tmz hold c_m, s_m and 2(m+1)z.
// ---------------------------------------------------------------------------
template <typename T, bool GRAD, bool HESS>
void channel(int l, T x, T y, T z, T rxy, const T* pk, const T* qk, const T* c, const T* s,
             const T* tmz, T* Y, T* DX, T* DY, T* DZ, T* const* DD) {
    T q2, q1, q0;                // Q_l^{m+2}, Q_l^{m+1}, Q_l^m
    T a2 = 0, a1 = 0, a0 = 0;    // same for l-1
    T b2 = 0, b1 = 0, b0 = 0;    // same for l-2
    T x2 = 0, y2 = 0, xy = 0;
    if (HESS) {
        x2 = x * x;
        y2 = y * y;
        xy = x * y;
    }

    // |m| = l                                             (:122-152)
    q2 = qk[l];
    T pq = q2 * pk[l];
    Y[-l] = pq * s[l];
    Y[+l] = pq * c[l];
    if (GRAD) {
        pq *= l;
        DX[-l] = pq * s[l - 1];
        DY[-l] = DX[l] = pq * c[l - 1];
        DY[l] = -DX[-l];
        DZ[-l] = 0;
        DZ[l] = 0;
        a2 = 0;
        if (HESS) {
            pq *= (l - 1);
            DD[XX][l] = pq * c[l - 2];
            DD[XX][-l] = pq * s[l - 2];
            DD[XY][l] = DD[YX][l] = DD[YY][-l] = -DD[XX][-l];
            DD[XY][-l] = DD[YX][-l] = DD[XX][l];
            DD[XZ][l] = DD[ZX][l] = 0.0;
            DD[XZ][-l] = DD[ZX][-l] = 0.0;
            DD[YY][l] = -DD[XX][l];
            DD[YZ][l] = DD[ZY][l] = 0.0;
            DD[YZ][-l] = DD[ZY][-l] = 0.0;
            DD[ZZ][l] = DD[ZZ][-l] = 0.0;
            b2 = 0.0;
        }
    }

    // |m| = l - 1                                         (:154-198)
    q1 = -z * q2;
    pq = q1 * pk[l - 1];
    Y[-l + 1] = pq * s[l - 1];
    Y[+l - 1] = pq * c[l - 1];
    if (GRAD) {
        pq *= (l - 1);
        DX[-l + 1] = pq * s[l - 2];
        DY[-l + 1] = DX[l - 1] = pq * c[l - 2];
        DY[l - 1] = -DX[-l + 1];
        a1 = qk[-1];
        T pdq = pk[l - 1] * (l + l - 1) * a1;
        DZ[-l + 1] = pdq * s[l - 1];
        DZ[l - 1] = pdq * c[l - 1];
        if (HESS) {
            pq *= (l - 2);
            if (l == 2) {
                DD[XX][l - 1] = 0;
                DD[XX][-l + 1] = 0;
            } else {
                DD[XX][l - 1] = pq * c[l - 3];
                DD[XX][-l + 1] = pq * s[l - 3];
            }
            DD[XY][l - 1] = DD[YX][l - 1] = DD[YY][-l + 1] = -DD[XX][-l + 1];
            DD[XY][-l + 1] = DD[YX][-l + 1] = DD[XX][l - 1];
            T t = -pk[l - 1] * (l - 1) * q2;
            DD[XZ][l - 1] = DD[ZX][l - 1] = t * c[l - 2];
            DD[XZ][-l + 1] = DD[ZX][-l + 1] = t * s[l - 2];
            DD[YY][l - 1] = -DD[XX][l - 1];
            DD[YZ][l - 1] = DD[ZY][l - 1] = -DD[XZ][-l + 1];
            DD[YZ][-l + 1] = DD[ZY][-l + 1] = DD[XZ][l - 1];
            DD[ZZ][l - 1] = DD[ZZ][-l + 1] = 0.0;
            b1 = 0.0;
        }
    }

    // l - 2 >= |m| >= 1; the reference splits this loop in two pieces with the
    // same body (:201-294 and :295-390), together they cover exactly this range.
    for (int m = l - 2; m > 0; --m) {
        q0 = qk[m] * (tmz[m] * q1 + rxy * q2);
        q2 = q1;
        q1 = q0;
        pq = q0 * pk[m];
        Y[-m] = pq * s[m];
        Y[+m] = pq * c[m];

        if (GRAD) {
            a0 = qk[m - l] * (tmz[m] * a1 + rxy * a2);
            a2 = a1;
            a1 = a0;

            pq *= m;
            T pqs = pq * s[m - 1], pqc = pq * c[m - 1];
            T pdq = pk[m] * a2;
            T pdqx = pdq * x;
            DX[-m] = (pdqx * s[m] + pqs);
            DX[+m] = (pdqx * c[m] + pqc);
            T pdqy = pdq * y;
            DY[-m] = (pdqy * s[m] + pqc);
            DY[m] = (pdqy * c[m] - pqs);
            pdq = pk[m] * (l + m) * a1;
            DZ[-m] = pdq * s[m];
            DZ[m] = pdq * c[m];

            if (HESS) {
                if (m == l - 2) {
                    b0 = qk[-l - 1];
                } else {
                    b0 = qk[m - 2 * l + 1] * (tmz[m] * b1 + rxy * b2);
                }

                pq /= m;
                // after the shift above a2 is Q_{l-1}^{m+1} and a1 is Q_{l-1}^m
                T pa_hi = pk[m] * a2;
                T pb2 = pk[m] * b2;
                T pb0 = pk[m] * b0;
                T pa_lo = pk[m] * a1;
                T pb1 = pk[m] * b1;

                T mmc = 0.0;
                T mms = 0.0;
                if (m != 1) {
                    mmc = m * (m - 1) * pq * c[m - 2];
                    mms = m * (m - 1) * pq * s[m - 2];
                }

                DD[XX][m] = pa_hi * c[m] + x2 * pb2 * c[m] + 2 * m * x * pa_hi * c[m - 1] + mmc;
                DD[XX][-m] = pa_hi * s[m] + x2 * pb2 * s[m] + 2 * m * x * pa_hi * s[m - 1] + mms;
                DD[YY][m] = pa_hi * c[m] + y2 * pb2 * c[m] - 2 * m * y * pa_hi * s[m - 1] - mmc;
                DD[YY][-m] = pa_hi * s[m] + y2 * pb2 * s[m] + 2 * m * y * pa_hi * c[m - 1] - mms;
                DD[ZZ][m] = (l + m) * (l + m - 1) * pb0 * c[m];
                DD[ZZ][-m] = (l + m) * (l + m - 1) * pb0 * s[m];

                DD[XY][m] = DD[YX][m] =
                    xy * pb2 * c[m] + y * pa_hi * m * c[m - 1] - x * pa_hi * m * s[m - 1] - mms;
                DD[XY][-m] = DD[YX][-m] =
                    xy * pb2 * s[m] + y * pa_hi * m * s[m - 1] + x * pa_hi * m * c[m - 1] + mmc;
                DD[XZ][m] = DD[ZX][m] =
                    x * (l + m) * pb1 * c[m] + (l + m) * pa_lo * m * c[m - 1];
                DD[XZ][-m] = DD[ZX][-m] =
                    x * (l + m) * pb1 * s[m] + (l + m) * pa_lo * m * s[m - 1];
                DD[YZ][m] = DD[ZY][m] =
                    y * (l + m) * pb1 * c[m] - (l + m) * pa_lo * m * s[m - 1];
                DD[YZ][-m] = DD[ZY][-m] =
                    y * (l + m) * pb1 * s[m] + (l + m) * pa_lo * m * c[m - 1];

                b2 = b1;
                b1 = b0;
            }
        }
    }

    // m = 0                                               (:392-426)
    q0 = qk[0] * (tmz[0] * q1 + rxy * q2);
    Y[0] = q0 * pk[0];
    if (GRAD) {
        a0 = qk[-l] * (tmz[0] * a1 + rxy * a2);
        DX[0] = pk[0] * x * a1;
        DY[0] = pk[0] * y * a1;
        DZ[0] = pk[0] * l * a0;
        if (HESS) {
            if (l == 2) {
                b0 = qk[-2 * l + 1];
            } else {
                b0 = qk[-2 * l + 1] * (tmz[0] * b1 + rxy * b2);
            }
            T pa1 = pk[0] * a1;
            T pb2 = pk[0] * b2;
            T pb0 = pk[0] * b0;
            T pb1 = pk[0] * b1;
            DD[XX][0] = pa1 + x2 * pb2;
            DD[YY][0] = pa1 + y2 * pb2;
            DD[ZZ][0] = (l) * (l - 1) * pb0;
            DD[XY][0] = DD[YX][0] = xy * pb2;
            DD[XZ][0] = DD[ZX][0] = x * l * pb1;
            DD[YZ][0] = DD[ZY][0] = y * l * pb1;
        }
    }
}

// ---------------------------------------------------------------------------
// Chain rule for evaluating the solid polynomials at (x, y, z)/r: Hessian
// first (it needs the uncorrected gradient), then gradient.
// templates.hpp:214-265 and :553-614. x, y, z are the already scaled
// coordinates, ir = 1/r.
// ---------------------------------------------------------------------------
template <typename T, bool HESS>
void unit_sphere_fixup(int ny, T x, T y, T z, T ir, T* DX, T* DY, T* DZ, T* const* DD) {
    for (int k = 0; k < ny; ++k) {
        T tmp = (DX[k] * x + DY[k] * y + DZ[k] * z);
        if (HESS) {
            T irsq = ir * ir;
            T tmpx = x * DD[XX][k] + y * DD[YX][k] + z * DD[ZX][k];
            T tmpy = x * DD[XY][k] + y * DD[YY][k] + z * DD[YZ][k];
            T tmpz = x * DD[XZ][k] + y * DD[YZ][k] + z * DD[ZZ][k];
            T tmp2 = x * x * DD[XX][k] + y * y * DD[YY][k] + z * z * DD[ZZ][k] +
                     2 * x * y * DD[XY][k] + 2 * x * z * DD[XZ][k] + 2 * y * z * DD[YZ][k];
            DD[XX][k] = (-2 * x * tmpx + DD[XX][k] + 3 * x * x * tmp - tmp - 2 * x * DX[k] +
                         x * x * tmp2) *
                        irsq;
            DD[YY][k] = (-2 * y * tmpy + DD[YY][k] + 3 * y * y * tmp - tmp - 2 * y * DY[k] +
                         y * y * tmp2) *
                        irsq;
            DD[ZZ][k] = (-2 * z * tmpz + DD[ZZ][k] + 3 * z * z * tmp - tmp - 2 * z * DZ[k] +
                         z * z * tmp2) *
                        irsq;
            DD[XY][k] = DD[YX][k] = (-x * tmpy - y * tmpx + DD[XY][k] + 3 * x * y * tmp -
                                     x * DY[k] - y * DX[k] + x * y * tmp2) *
                                    irsq;
            DD[XZ][k] = DD[ZX][k] = (-x * tmpz - z * tmpx + DD[XZ][k] + 3 * x * z * tmp -
                                     x * DZ[k] - z * DX[k] + x * z * tmp2) *
                                    irsq;
            DD[ZY][k] = DD[YZ][k] = (-z * tmpy - y * tmpz + DD[ZY][k] + 3 * y * z * tmp -
                                     z * DY[k] - y * DZ[k] + y * z * tmp2) *
                                    irsq;
        }
        DX[k] = (DX[k] - x * tmp) * ir;
        DY[k] = (DY[k] - y * tmp) * ir;
        DZ[k] = (DZ[k] - z * tmp) * ir;
    }
}

// Which l are evaluated in closed form. sphericart.cpp:45-92 (and :428-475 for
// the solid class): without Hessians everything up to l = 6; with Hessians only
// l <= 1, the recursion takes over from l = 2 -- for the values and gradients
// returned alongside the Hessians too.
inline int hardcoded_limit(int L, bool hess) {
    const int cap = hess ? 1 : 6;
    return L < cap ? L : cap;
}

// ---------------------------------------------------------------------------
// One point. templates.hpp:99-267 (closed form only) and :333-615 (closed
// form + recursion); the two coincide on their common part. H is the largest
// l evaluated in closed form; c/s/tmz are scratch of L+1 entries each.
// ---------------------------------------------------------------------------
template <typename T, bool GRAD, bool HESS, bool NORM>
void one_sample(const T* p, int L, int H, const T* pref, T* c, T* s, T* tmz, T* sph, T* dsph,
                T* ddsph) {
    const int ny = (L + 1) * (L + 1);
    const int nq = (L + 1) * (L + 2) / 2;

    T x = p[0], y = p[1], z = p[2];
    T x2 = x * x, y2 = y * y, z2 = z * z;
    T ir = 0.0;
    if (NORM) {
        ir = 1 / std::sqrt(x2 + y2 + z2);
        x *= ir;
        y *= ir;
        z *= ir;
        x2 = x * x;
        y2 = y * y;
        z2 = z * z;
    }
    T rxy = x2 + y2;

    T* DX = nullptr;
    T* DY = nullptr;
    T* DZ = nullptr;
    T* DD[9] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};

    low_values<T>(H, x, y, z, x2, y2, z2, sph);
    if (GRAD) {
        DX = dsph;
        DY = DX + ny;
        DZ = DY + ny;
        low_gradients<T>(H, x, y, z, x2, y2, z2, sph, DX, DY, DZ);
    }
    if (HESS) {
        // macros.hpp:56-131: all second derivatives of l = 0, 1 vanish
        for (int a = 0; a < 9; ++a) {
            DD[a] = ddsph + a * ny;
            for (int k = 0; k < (H + 1) * (H + 1); ++k) {
                DD[a][k] = K(0.0);
            }
        }
    }

    if (L > H) {
        // templates.hpp:451-466
        T twoz = z + z;
        tmz[0] = twoz;
        c[0] = 1.0;
        s[0] = 0.0;
        for (int m = 1; m < L + 1; ++m) {
            c[m] = c[m - 1] * x - s[m - 1] * y;
            s[m] = c[m - 1] * y + s[m - 1] * x;
            tmz[m] = tmz[m - 1] + twoz;
        }

        const T* pq = pref + nq;
        for (int l = H + 1; l <= L; ++l) {
            const int mid = l * (l + 1);
            const int tri = l * (l + 1) / 2;
            T* dd[9];
            for (int a = 0; a < 9; ++a) {
                dd[a] = HESS ? DD[a] + mid : nullptr;
            }
            channel<T, GRAD, HESS>(l, x, y, z, rxy, pref + tri, pq + tri, c, s, tmz, sph + mid,
                                   GRAD ? DX + mid : nullptr, GRAD ? DY + mid : nullptr,
                                   GRAD ? DZ + mid : nullptr, dd);
        }
    }

    if (GRAD && NORM) {
        unit_sphere_fixup<T, HESS>(ny, x, y, z, ir, DX, DY, DZ, DD);
    }
}

// Sample loop. templates.hpp:308-330 and :677-709.
template <typename T, bool GRAD, bool HESS, bool NORM>
void many_samples(const T* xyz, size_t n, int L, int H, const T* pref, T* sph, T* dsph, T* ddsph) {
    const size_t ny = static_cast<size_t>(L + 1) * (L + 1);
#pragma omp parallel
    {
        std::vector<T> scratch(3 * static_cast<size_t>(L + 1));
        T* c = scratch.data();
        T* s = c + (L + 1);
        T* tmz = s + (L + 1);
#pragma omp for
        for (int64_t i = 0; i < static_cast<int64_t>(n); ++i) {
            one_sample<T, GRAD, HESS, NORM>(xyz + 3 * i, L, H, pref, c, s, tmz, sph + i * ny,
                                            GRAD ? dsph + 3 * i * ny : nullptr,
                                            HESS ? ddsph + 9 * i * ny : nullptr);
        }
    }
}

// mode: 0 values, 1 values + gradients, 2 values + gradients + Hessians.
// hard < 0 picks the reference's own rule, hard >= 1 forces that closed-form
// limit (used for the route-consistency check).
template <typename T>
int run(const T* xyz, size_t n, int L, int normalized, int mode, int hard, T* sph, T* dsph,
        T* ddsph) {
    if (L < 0 || mode < 0 || mode > 2) return 2;
    if (n == 0) return 0;
    if (!xyz || !sph || (mode >= 1 && !dsph) || (mode >= 2 && !ddsph)) return 3;
    int H = hardcoded_limit(L, mode == 2);
    if (hard >= 0) {
        if (hard > 6 || hard > L || (mode == 2 && hard > 1) || (hard < 1 && L > hard)) return 4;
        H = hard;
    }
    std::vector<T> pref(static_cast<size_t>(L + 1) * (L + 2));
    prefactors<T>(L, pref.data());
    const bool nrm = normalized != 0;
    if (mode == 0) {
        nrm ? many_samples<T, false, false, true>(xyz, n, L, H, pref.data(), sph, dsph, ddsph)
            : many_samples<T, false, false, false>(xyz, n, L, H, pref.data(), sph, dsph, ddsph);
    } else if (mode == 1) {
        nrm ? many_samples<T, true, false, true>(xyz, n, L, H, pref.data(), sph, dsph, ddsph)
            : many_samples<T, true, false, false>(xyz, n, L, H, pref.data(), sph, dsph, ddsph);
    } else {
        nrm ? many_samples<T, true, true, true>(xyz, n, L, H, pref.data(), sph, dsph, ddsph)
            : many_samples<T, true, true, false>(xyz, n, L, H, pref.data(), sph, dsph, ddsph);
    }
    return 0;
}

#undef K

// xyz_grad[i][a] = sum_k dsph[i][a][k] * sph_grad[i][k]
template <typename T>
void backward(const T* dsph, const T* sph_grad, size_t n, int n_total, T* xyz_grad) {
    for (size_t i = 0; i < n; ++i) {
        for (int a = 0; a < 3; ++a) {
            T sum = 0;
            for (int k = 0; k < n_total; ++k) {
                sum += dsph[(i * 3 + a) * n_total + k] * sph_grad[i * n_total + k];
            }
            xyz_grad[i * 3 + a] = sum;
        }
    }
}

// xyz_grad[i][b] = sum_a sum_k ddsph[i][a][b][k] * dsph_grad[i][a][k]
template <typename T>
void backward_second(const T* ddsph, const T* dsph_grad, size_t n, int n_total, T* xyz_grad) {
    for (size_t i = 0; i < n; ++i) {
        for (int b = 0; b < 3; ++b) {
            T sum = 0;
            for (int a = 0; a < 3; ++a) {
                for (int k = 0; k < n_total; ++k) {
                    sum += ddsph[((i * 3 + a) * 3 + b) * n_total + k] *
                           dsph_grad[(i * 3 + a) * n_total + k];
                }
            }
            xyz_grad[i * 3 + b] = sum;
        }
    }
}

} // namespace

extern "C" {

int sphx_oracle_compute_f64(const double* xyz, size_t n, int l_max, int normalized, int mode,
                            double* sph, double* dsph, double* ddsph) {
    return run<double>(xyz, n, l_max, normalized, mode, -1, sph, dsph, ddsph);
}

int sphx_oracle_compute_f32(const float* xyz, size_t n, int l_max, int normalized, int mode,
                            float* sph, float* dsph, float* ddsph) {
    return run<float>(xyz, n, l_max, normalized, mode, -1, sph, dsph, ddsph);
}

// Recursion route with only l <= 1 in closed form (values / gradients only).
int sphx_oracle_recursion_route_f64(const double* xyz, size_t n, int l_max, int normalized,
                                    int mode, double* sph, double* dsph) {
    if (l_max < 2 || mode > 1) return 2;
    return run<double>(xyz, n, l_max, normalized, mode, 1, sph, dsph, nullptr);
}

int sphx_oracle_recursion_route_f32(const float* xyz, size_t n, int l_max, int normalized,
                                    int mode, float* sph, float* dsph) {
    if (l_max < 2 || mode > 1) return 2;
    return run<float>(xyz, n, l_max, normalized, mode, 1, sph, dsph, nullptr);
}

void sphx_oracle_prefactors_f64(int l_max, double* out) { prefactors<double>(l_max, out); }

void sphx_oracle_prefactors_f32(int l_max, float* out) { prefactors<float>(l_max, out); }

int sphx_oracle_hardcoded_limit(int l_max, int with_hessians) {
    return hardcoded_limit(l_max, with_hessians != 0);
}

void sphx_oracle_backward_f64(const double* dsph, const double* sph_grad, size_t n, int n_total,
                              double* xyz_grad) {
    backward<double>(dsph, sph_grad, n, n_total, xyz_grad);
}

void sphx_oracle_backward_f32(const float* dsph, const float* sph_grad, size_t n, int n_total,
                              float* xyz_grad) {
    backward<float>(dsph, sph_grad, n, n_total, xyz_grad);
}

void sphx_oracle_backward_second_f64(const double* ddsph, const double* dsph_grad, size_t n,
                                     int n_total, double* xyz_grad) {
    backward_second<double>(ddsph, dsph_grad, n, n_total, xyz_grad);
}

void sphx_oracle_backward_second_f32(const float* ddsph, const float* dsph_grad, size_t n,
                                     int n_total, float* xyz_grad) {
    backward_second<float>(ddsph, dsph_grad, n, n_total, xyz_grad);
}

int sphx_oracle_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

} // extern "C"
