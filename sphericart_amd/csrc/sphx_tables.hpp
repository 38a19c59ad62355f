// Host-side prefactor tables: F_l^m (normalisation of Y_l^m, with the 1/sqrt(2)
// of m = 0 folded in) and the constants of the downward-in-m Q_l^m recursion.
// Both are triangular, entry (l, m) at l(l+1)/2 + m, and depend on (l, m) only,
// so the table for SPHX_TABLE_LMAX contains the table of every smaller l_max
// as a prefix of each block.
#pragma once

#include <vector>

namespace sphx {

struct HostTables {
    // [0, n) holds F, [n, 2n) holds the Q constants, n = (LMAX+1)(LMAX+2)/2
    std::vector<float> f32;
    std::vector<double> f64;
};

// Built on first use, in the arithmetic type of each table, with the
// recurrences of the reference (sphericart/include/templates.hpp:54-97).
const HostTables& host_tables();

} // namespace sphx
