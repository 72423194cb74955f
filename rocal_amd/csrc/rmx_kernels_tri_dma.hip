// K2t streaming path: picks the instance of rmx_resize_tri_dma_kernel (rmx_kernels_tri_dma_impl.h) for a batch. The instances
// live in translation units of their own (rmx_kernels_tri_dma_2 / _4 / _8_nchw / _8_nhwc.hip), which compile side by side.
#include "rmx_launch.h"

namespace rmx {

KernelFn tdma_unit_2_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_2_nhwc(int dtype, bool norm, bool quant);
KernelFn tdma_unit_4_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_4_nhwc(int dtype, bool norm, bool quant);
KernelFn tdma_unit_8_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_8_nhwc(int dtype, bool norm, bool quant);

// rows_in_flight: 2 when the host has established that output rows two apart never read the same source row, 8 when some
// sample grows vertically, else 4
KernelFn select_resize_tri_dma_kernel(int dtype, int layout, bool norm, bool quant, int rows_in_flight, const char **name) {
    *name = "rmx_resize_tri_dma_kernel";
    const bool planar = layout == RMX_NCHW;
    if (rows_in_flight == 2) return planar ? tdma_unit_2_nchw(dtype, norm, quant) : tdma_unit_2_nhwc(dtype, norm, quant);
    if (rows_in_flight == 8) return planar ? tdma_unit_8_nchw(dtype, norm, quant) : tdma_unit_8_nhwc(dtype, norm, quant);
    return planar ? tdma_unit_4_nchw(dtype, norm, quant) : tdma_unit_4_nhwc(dtype, norm, quant);
}

}  // namespace rmx
