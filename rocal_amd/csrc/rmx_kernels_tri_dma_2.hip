// K2t streaming path, instances with 2 accumulator sets (see rmx_kernels_tri_dma_impl.h).
#include "rmx_kernels_tri_dma_impl.h"

namespace rmx {
RMX_TDMA_UNIT(2, RMX_NCHW, tdma_unit_2_nchw)
RMX_TDMA_UNIT(2, RMX_NHWC, tdma_unit_2_nhwc)
}  // namespace rmx
