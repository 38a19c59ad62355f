// recursion_kernel computing in float64 for float arrays, values, gradients and second derivatives: a translation unit
// of its own, so that the kernels of the library compile side by side.
#include "sphx_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_wide<2>(const Plan&, bool, const float*, float*, float*, float*, hipStream_t);
template hipError_t upload_wide_tables<2>(const HostTables&);

} // namespace sphx
