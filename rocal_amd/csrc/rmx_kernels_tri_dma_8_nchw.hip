// K2t streaming path, instances with 8 accumulator sets (see rmx_kernels_tri_dma_impl.h).
#include "rmx_kernels_tri_dma_impl.h"

namespace rmx {
RMX_TDMA_UNIT(8, RMX_NCHW, tdma_unit_8_nchw)
}  // namespace rmx
