// extern "C" doorways onto the reference's own in-tree HIP kernels, so tests can call them
// through ctypes without relying on C++ name mangling. Compiled together with
// <reference>/rocAL/rocAL_hip/rocal_hip_kernels.cpp into oracle/_ref/ (test infrastructure).
#include <hip/hip_runtime.h>
#include <cstddef>
#include "rocal_hip_kernels.h"

extern "C" {

// diagnostics: name of an error code, and the launch error left behind by the last call
const char *ref_error_name(int code) { return hipGetErrorName((hipError_t)code); }

// rocAL/rocAL_hip/rocal_hip_kernels.cpp:591-645; all pointer arrays must be device-readable.
int ref_resize_tensor(void *stream, void *src, void *dst, unsigned batch, size_t *src_w, size_t *src_h,
                      size_t *dst_w, size_t *dst_h, size_t *src_h_stride, size_t *src_img_offset,
                      unsigned channels, size_t max_src_w, size_t max_src_h, size_t max_dst_w,
                      size_t max_dst_h) {
    HipExecResizeTensor((hipStream_t)stream, src, dst, batch, src_w, src_h, dst_w, dst_h, src_h_stride,
                        src_img_offset, channels, max_src_w, max_src_h, max_dst_w, max_dst_h);
    hipError_t launch = hipGetLastError();
    hipError_t sync = hipStreamSynchronize((hipStream_t)stream);
    return launch != hipSuccess ? (int)launch : (int)sync;
}

// rocAL/rocAL_hip/rocal_hip_kernels.cpp:219-309
int ref_copy_int8_to_tensor(void *stream, const void *src, void *dst, int nchw_out, unsigned n, unsigned c,
                            unsigned h, unsigned w, const float *mul, const float *add, unsigned reverse,
                            unsigned fp16) {
    if (nchw_out)
        HipExecCopyInt8ToNCHW((hipStream_t)stream, src, dst, 0, n, c, h, w, mul[0], mul[1], mul[2], add[0],
                              add[1], add[2], reverse, fp16);
    else
        HipExecCopyInt8ToNHWC((hipStream_t)stream, src, dst, 0, n, c, h, w, mul[0], mul[1], mul[2], add[0],
                              add[1], add[2], reverse, fp16);
    hipError_t launch = hipGetLastError();
    hipError_t sync = hipStreamSynchronize((hipStream_t)stream);
    return launch != hipSuccess ? (int)launch : (int)sync;
}
}
