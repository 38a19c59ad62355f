// The fused product in float: a translation unit of its own, so that the kernels of the library compile side by
// side.
#include "sphx_vjp_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_vjp<float>(const VjpPlan&, int, bool, const float*, const float*, float*, int, hipStream_t);
template hipError_t upload_vjp_tables<float>(const HostTables&);

} // namespace sphx
