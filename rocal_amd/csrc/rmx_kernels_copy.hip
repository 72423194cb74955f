// Plain streaming copy (16 bytes per lane per step): the box's copy ceiling and the
// calibration kernel for rocprof's FETCH_SIZE / WRITE_SIZE counters.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

__global__ void __launch_bounds__(256) rmx_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n16; i += stride) dst[i] = src[i];
}

void launch_copy(hipStream_t stream, const void *src, void *dst, size_t nbytes, int num_cus) {
    const size_t n16 = nbytes / 16;
    size_t blocks = (n16 + 255) / 256;
    const size_t cap = (size_t)num_cus * 4;  // 4 resident workgroups per CU measured best for large copies
    if (blocks > cap) blocks = cap;
    if (blocks == 0) return;
    hipLaunchKernelGGL(rmx_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint4 *)src, (uint4 *)dst, n16);
}

}  // namespace rmx
