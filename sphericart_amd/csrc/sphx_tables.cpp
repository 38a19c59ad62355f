#include "sphx_tables.hpp"

#include <cmath>
#include <cstring>

#include "../../include/sphx_launch.h"

namespace sphx {

namespace {

// sphericart/include/templates.hpp:54-97, written for two separate blocks.
// Every operation is done in T: the float table reproduces the reference's
// float roundings, including its underflow to zero from l ~ 20 and the
// overflow of (2l-1)!! at l = 29.
template <typename T> void fill(int l_max, T* F, T* Q) {
    const T pi = static_cast<T>(3.141592653589793238462643383279502884L);
    const T inv_sqrt_2 = static_cast<T>(0.707106781186547524400844362104849039L);
    for (int l = 0; l <= l_max; ++l) {
        T* row = F + l * (l + 1) / 2;
        T ratio = (2 * l + 1) / (2 * pi);
        row[0] = std::sqrt(ratio) * inv_sqrt_2;
        for (int m = 1; m <= l; ++m) {
            ratio *= static_cast<T>(1.0) / (l * (l + 1) + m * (1 - m));
            const T root = std::sqrt(ratio);
            row[m] = (m & 1) ? -root : root;
        }
    }
    Q[0] = 1;
    for (int l = 1; l <= l_max; ++l) {
        T* row = Q + l * (l + 1) / 2;
        const T above = row[-1]; // Q_{l-1}^{l-1}, the last entry of the previous row
        row[l] = -(2 * l - 1) * above;
        for (int m = l - 1; m >= 0; --m) {
            row[m] = static_cast<T>(-1.0) / ((l + m + 1) * (l - m));
        }
    }
}

} // namespace

const HostTables& host_tables() {
    static const HostTables tables = [] {
        HostTables t;
        const int n = (SPHX_TABLE_LMAX + 1) * (SPHX_TABLE_LMAX + 2) / 2;
        t.f32.resize(2 * n);
        t.f64.resize(2 * n);
        fill<float>(SPHX_TABLE_LMAX, t.f32.data(), t.f32.data() + n);
        fill<double>(SPHX_TABLE_LMAX, t.f64.data(), t.f64.data() + n);
        return t;
    }();
    return tables;
}

} // namespace sphx

namespace {

template <typename T> int copy_prefix(const std::vector<T>& table, int l_max, T* out) {
    if (l_max < 0 || out == nullptr) return SPHX_ERR_ARGUMENT;
    if (l_max > SPHX_TABLE_LMAX) return SPHX_ERR_UNSUPPORTED;
    const size_t full = table.size() / 2;
    const size_t n = static_cast<size_t>(l_max + 1) * (l_max + 2) / 2;
    std::memcpy(out, table.data(), n * sizeof(T));
    std::memcpy(out + n, table.data() + full, n * sizeof(T));
    return SPHX_OK;
}

} // namespace

extern "C" {

int sphx_prefactors_f32(int l_max, float* out) {
    return copy_prefix<float>(sphx::host_tables().f32, l_max, out);
}

int sphx_prefactors_f64(int l_max, double* out) {
    return copy_prefix<double>(sphx::host_tables().f64, l_max, out);
}

} // extern "C"
