// K2 general path, instantiations for one destination type and layout (see rmx_kernels_resize_impl.h).
#include "rmx_kernels_resize_impl.h"

namespace rmx {
RMX_RESIZE_UNIT(uint8_t, RMX_NCHW, resize_unit_u8_nchw)
}  // namespace rmx
