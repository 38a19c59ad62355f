// The forward kernels in double, values, gradients and second derivatives: a translation unit of its own, so that
// the kernels of the library compile side by side.
#include "sphx_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_forward<double, 2>(const Plan&, const DeviceState&, bool, const double*, double*, double*, double*,
                                             hipStream_t);
template hipError_t upload_forward_tables<double, 2>(const HostTables&, const double**, const double**);

} // namespace sphx
