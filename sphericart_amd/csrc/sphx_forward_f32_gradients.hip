// The forward kernels in float, values and gradients: a translation unit of its own, so that
// the kernels of the library compile side by side.
#include "sphx_dispatch.hpp"

namespace sphx {

template hipError_t dispatch_forward<float, 1>(const Plan&, const DeviceState&, bool, const float*, float*, float*, float*,
                                             hipStream_t);
template hipError_t upload_forward_tables<float, 1>(const HostTables&, const float**, const float**);

} // namespace sphx
