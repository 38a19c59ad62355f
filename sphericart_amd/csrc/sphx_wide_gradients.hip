// recursion_kernel computing in float64 for float arrays, values and gradients: a translation unit
// of its own, so that the kernels of the library compile side by side.
#include "sphx_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_wide<1>(const Plan&, bool, const float*, float*, float*, float*, hipStream_t);
template hipError_t upload_wide_tables<1>(const HostTables&);

} // namespace sphx
