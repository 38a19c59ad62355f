// The fused product in double: a translation unit of its own, so that the kernels of the library compile side by
// side.
#include "sphx_vjp_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_vjp<double>(const VjpPlan&, int, bool, const double*, const double*, double*, int, hipStream_t);
template hipError_t upload_vjp_tables<double>(const HostTables&);

} // namespace sphx
