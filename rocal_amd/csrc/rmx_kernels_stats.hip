// Normalize (mean / standard deviation over the image axes of each sample): the two kernels in front of the streaming pass.
//   rmx_stats_reduce_kernel    one wavefront per (sample, strip of rows): per-channel sum and sum of squares of the
//                              sample's window as exact integers (bytes: no rounding, so the order of the additions does not
//                              matter), reduced across the wavefront and added to the sample's six 64-bit counters;
//   rmx_stats_finalize_kernel  one thread per (sample, channel): mean and population standard deviation in double from the
//                              exact integer moments, then the FMA constants of the streaming pass written into the sample's row
//                              of the parameter table:  a = scale / sigma,  b = shift - mean * a  (sigma = 0: a = 0, b = shift).
// The streaming pass itself is the CropMirrorNormalize kernel (one fp32 FMA per value), reading those rows.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

__global__ void __launch_bounds__(256) rmx_stats_zero_kernel(unsigned long long *counters, int count) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) counters[i] = 0ull;
}

__global__ void __launch_bounds__(256) rmx_stats_reduce_kernel(RmxKArgs a, unsigned long long *counters) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (blockDim.x / RMX_WAVE) + threadIdx.x / RMX_WAVE;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, strip;
    wave_to_sample(a, wave, s, strip, false);  // no XCD renumbering in this kernel: batch order keeps the address stream contiguous
    const RmxSample &P = a.table[s];
    const int w = P.dst_w, h = P.dst_h, x1 = P.src_x, y1 = P.src_y;
    const int r0 = strip * a.aux0;
    if (r0 >= h || w <= 0) return;
    const int r1 = min(r0 + a.aux0, h);
    uint32_t row_stride32;
    const uint8_t *simg = sample_base(a, s, row_stride32);
    const uint8_t *buf_end = a.src + a.src_bytes;
    // per lane: at most 8 rows x (w / 512 + 1) groups of 8 pixels: sums stay far below 2^32
    uint32_t sum[3] = {0, 0, 0}, sq[3] = {0, 0, 0};
    const int groups = (w + PX - 1) / PX;
    for (int r = r0; r < r1; r++) {
        const uint8_t *row = simg + (size_t)(y1 + r) * row_stride32 + (size_t)x1 * 3;
        for (int g = lane; g < groups; g += RMX_WAVE) {
            const int cnt = min(PX, w - g * PX);
            uint32_t d[6];
            load_realigned<7>(row + (size_t)g * PX * 3, buf_end, d);
#pragma unroll
            for (int k = 0; k < PX; k++) {
                if (k < cnt) {
#pragma unroll
                    for (int c = 0; c < 3; c++) {
                        const int byte = 3 * k + c;
                        const uint32_t v = (d[byte >> 2] >> (8 * (byte & 3))) & 0xffu;
                        sum[c] += v;
                        sq[c] += v * v;
                    }
                }
            }
        }
    }
#pragma unroll
    for (int c = 0; c < 3; c++) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            sum[c] += __shfl_xor(sum[c], off, RMX_WAVE);
            sq[c] += __shfl_xor(sq[c], off, RMX_WAVE);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            atomicAdd(&counters[(size_t)s * 6 + c], (unsigned long long)sum[c]);
            atomicAdd(&counters[(size_t)s * 6 + 3 + c], (unsigned long long)sq[c]);
        }
    }
}

// mode bit 0: the mean is computed (else given), bit 1: the standard deviation is computed (else given); per_channel: one
// statistic per channel (axes H, W) or one for the whole sample (axes H, W, C). given_mean / given_std hold 3 values per sample.
__global__ void __launch_bounds__(256) rmx_stats_finalize_kernel(RmxSample *table, const unsigned long long *counters, const float *given, int n,
                                                                 int mode, int per_channel, float scale, float shift) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n * 3) return;
    const int s = i / 3, c = i - 3 * s;
    RmxSample &P = table[s];
    const unsigned long long *cn = counters + (size_t)s * 6;
    double cnt = (double)P.dst_w * (double)P.dst_h, sum = (double)cn[c], sq = (double)cn[3 + c];
    if (!per_channel) {
        cnt *= 3.0;
        sum = (double)(cn[0] + cn[1] + cn[2]);
        sq = (double)(cn[3] + cn[4] + cn[5]);
    }
    float mean = given[(size_t)s * 6 + c], sigma = given[(size_t)s * 6 + 3 + c];
    if (cnt > 0.0) {
        const double m = (mode & 1) ? sum / cnt : (double)mean;
        if (mode & 1) mean = (float)m;
        if (mode & 2) {
            // sum of (x - m)^2 = sq - 2 m sum + cnt m^2, every term exact or correctly rounded in double
            double var = (sq - 2.0 * m * sum + cnt * m * m) / cnt;
            if (var < 0.0) var = 0.0;
            sigma = (float)__builtin_sqrt(var);
        }
    }
    const float a = sigma != 0.0f ? scale / sigma : 0.0f;
    P.scale[c] = a;
    P.bias[c] = __builtin_fmaf(-mean, a, shift);
}

void launch_stats(hipStream_t stream, const RmxKArgs &a, unsigned long long *counters, RmxSample *table, const float *given, int mode, int per_channel,
                  float scale, float shift, bool reduce) {
    if (reduce) {
        const int count = a.n * 6;
        hipLaunchKernelGGL(rmx_stats_zero_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, counters, count);
        const uint32_t waves = (uint32_t)a.n * (uint32_t)a.strips;
        hipLaunchKernelGGL(rmx_stats_reduce_kernel, dim3((waves + 3) / 4), dim3(256), 0, stream, a, counters);
    }
    hipLaunchKernelGGL(rmx_stats_finalize_kernel, dim3((a.n * 3 + 255) / 256), dim3(256), 0, stream, table, counters, given, a.n, mode, per_channel, scale,
                       shift);
}

}  // namespace rmx
