// Host-side kernel selection: each kernel family exports a selector that maps the static
// node configuration to one template instantiation.
#pragma once
#include "rmx_common.h"

namespace rmx {
typedef void (*KernelFn)(RmxKArgs);

KernelFn select_cmn_kernel(int dtype, int layout, bool norm, int mode, const char **name);
KernelFn select_resize_linear_kernel(int dtype, int layout, bool norm, bool quant, int chain, const char **name);
KernelFn select_resize_fast_kernel(int dtype, int layout, bool norm, bool quant, int chain, const char **name);
KernelFn select_resize_dma_kernel(int dtype, int layout, bool norm, bool quant, int chain, bool aligned, const char **name);
KernelFn select_resize_nearest_kernel(int dtype, int layout, bool norm, bool quant, const char **name);
KernelFn select_resize_tri_kernel(int dtype, int layout, bool norm, bool quant, const char **name);
KernelFn select_resize_tri_down_kernel(int dtype, int layout, bool norm, bool quant, int columns_per_lane, const char **name);
KernelFn select_resize_tri_dma_kernel(int dtype, int layout, bool norm, bool quant, int rows_in_flight, const char **name);
KernelFn select_color_kernel(int kind, int dtype, int layout, int mode, const char **name);
KernelFn select_point_kernel(int kind, int dtype, int layout, int mode, const char **name);
KernelFn select_transpose_kernel(int dtype, int layout, const char **name);
KernelFn select_warp_kernel(int interp, int dtype, int layout, bool raw, const char **name);
// LDS pitch, in 16-byte pieces, at which the raw form of the warp kernel stages every box that fits it
#ifndef RMX_WARP_RAW_PIECES
#define RMX_WARP_RAW_PIECES 11
#endif
constexpr int kWarpRawPieces = RMX_WARP_RAW_PIECES;
// Normalize: (reduce: zero + per-sample integer moments,) then the FMA constants into the rows of `table` (device memory)
void launch_stats(hipStream_t stream, const RmxKArgs &a, unsigned long long *counters, RmxSample *table, const float *given, int mode, int per_channel,
                  float scale, float shift, bool reduce);
void launch_copy(hipStream_t stream, const void *src, void *dst, size_t nbytes, int num_cus);
// mode 0 copy, 1 read only, 2 write only; groups_per_cu 0 = the default (16)
void launch_stream(hipStream_t stream, int mode, const void *src, void *dst, size_t nbytes, int num_cus, int groups_per_cu);
}  // namespace rmx
