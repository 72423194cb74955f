// K2 general path: selector over the per-type translation units (kernel in rmx_kernels_resize_impl.h).
#include "rmx_launch.h"

namespace rmx {

KernelFn resize_unit_f32_nchw(bool nearest, bool norm, bool quant, int chain);
KernelFn resize_unit_f16_nchw(bool nearest, bool norm, bool quant, int chain);
KernelFn resize_unit_u8_nchw(bool nearest, bool norm, bool quant, int chain);
KernelFn resize_unit_f32_nhwc(bool nearest, bool norm, bool quant, int chain);
KernelFn resize_unit_f16_nhwc(bool nearest, bool norm, bool quant, int chain);
KernelFn resize_unit_u8_nhwc(bool nearest, bool norm, bool quant, int chain);

static KernelFn pick(bool nearest, int dtype, int layout, bool norm, bool quant, int chain) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return resize_unit_f32_nchw(nearest, norm, quant, chain);
            case RMX_FP16: return resize_unit_f16_nchw(nearest, norm, quant, chain);
            default: return resize_unit_u8_nchw(nearest, norm, quant, chain);
        }
    }
    switch (dtype) {
        case RMX_FP32: return resize_unit_f32_nhwc(nearest, norm, quant, chain);
        case RMX_FP16: return resize_unit_f16_nhwc(nearest, norm, quant, chain);
        default: return resize_unit_u8_nhwc(nearest, norm, quant, chain);
    }
}

KernelFn select_resize_linear_kernel(int dtype, int layout, bool norm, bool quant, int chain, const char **name) {
    *name = "rmx_resize_kernel";
    return pick(false, dtype, layout, norm, quant, chain);
}

KernelFn select_resize_nearest_kernel(int dtype, int layout, bool norm, bool quant, const char **name) {
    *name = "rmx_resize_kernel";
    return pick(true, dtype, layout, norm, quant, 0);
}

}  // namespace rmx
