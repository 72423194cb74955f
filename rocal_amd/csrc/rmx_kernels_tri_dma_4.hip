// K2t streaming path, instances with 4 accumulator sets (see rmx_kernels_tri_dma_impl.h).
#include "rmx_kernels_tri_dma_impl.h"

namespace rmx {
RMX_TDMA_UNIT(4, RMX_NCHW, tdma_unit_4_nchw)
RMX_TDMA_UNIT(4, RMX_NHWC, tdma_unit_4_nhwc)
}  // namespace rmx
