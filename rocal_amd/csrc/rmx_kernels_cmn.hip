// K1: crop + horizontal/vertical flip + per-channel FMA + layout transpose + cast, one pass.
// Serves CropMirrorNormalize, Crop and Flip (u8 NHWC in; f32/f16/u8, NCHW/NHWC out).
//
// Scheduling: one wavefront owns a strip of output rows of one sample. Inside a step the
// wave covers G = 64/L rows at once, L = lanes per row, each lane producing 8 adjacent
// pixels: a 28-byte realigned read of packed RGB in, three 128-bit planar stores out (fp16).
// HBM-bound: 3 bytes read and 3*sizeof(T) written per output pixel, no reuse.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

template <typename T, int LAYOUT, bool NORM>
__global__ void __launch_bounds__(256) rmx_cmn_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    const uint32_t nblocks = gridDim.x;
    uint32_t wave = xcd_swizzle(blockIdx.x, nblocks) * (blockDim.x / RMX_WAVE) + (threadIdx.x / RMX_WAVE);
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    const int s = (int)(wave / (uint32_t)a.strips);
    const int strip = (int)(wave % (uint32_t)a.strips);
    const RmxSample &P = a.table[s];

    const int cw = P.dst_w, ch = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= ch) return;
    const int r1 = min(r0 + srows, ch);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;
    const bool vf = (P.flags & RMX_S_VFLIP) != 0;
    const int x1 = P.src_x, y1 = P.src_y;

    const size_t row_stride = (size_t)a.src_w * 3;
    const uint8_t *simg = a.src + (size_t)s * a.src_h * row_stride;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    for (int xt = 0; xt < cw; xt += RMX_WAVE * PX) {
        const int tw = min(cw - xt, RMX_WAVE * PX);
        const int L = (tw + PX - 1) / PX;  // lanes per row, <= 64
        const int G = RMX_WAVE / L;        // rows per step
        const int lr = lane / L;
        const int g = lane - lr * L;
        const int gx = xt + g * PX;               // first output column of this lane's group
        const int cnt = min(PX, cw - gx);         // valid pixels in the group
        const bool active = lr < G;
        // source column of group pixel 0 (mirror reads the mirrored run and reverses it)
        const int sx0 = x1 + (hf ? (cw - gx - cnt) : gx);
        for (int r = r0 + lr; r < r1 && active; r += G) {
            const int sy = y1 + (vf ? (ch - 1 - r) : r);
            const uint8_t *p = simg + (size_t)sy * row_stride + (size_t)sx0 * 3;
            uint32_t w[6];
            load_realigned<7>(p, buf_end, w);
            float v[3][PX];
            unpack8(w, v);
            if constexpr (NORM) {
#pragma unroll
                for (int c = 0; c < 3; c++)
#pragma unroll
                    for (int k = 0; k < PX; k++) v[c][k] = __builtin_fmaf(v[c][k], sc[c], bi[c]);
            }
            store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, gx, cnt, v, hf);
        }
    }
}

#define RMX_CMN_INST(T, LAY, NORM) template __global__ void rmx_cmn_kernel<T, LAY, NORM>(RmxKArgs);
RMX_CMN_INST(float, RMX_NCHW, true)
RMX_CMN_INST(float, RMX_NHWC, true)
RMX_CMN_INST(__half, RMX_NCHW, true)
RMX_CMN_INST(__half, RMX_NHWC, true)
RMX_CMN_INST(uint8_t, RMX_NCHW, true)
RMX_CMN_INST(uint8_t, RMX_NHWC, true)
RMX_CMN_INST(float, RMX_NCHW, false)
RMX_CMN_INST(float, RMX_NHWC, false)
RMX_CMN_INST(__half, RMX_NCHW, false)
RMX_CMN_INST(__half, RMX_NHWC, false)
RMX_CMN_INST(uint8_t, RMX_NCHW, false)
RMX_CMN_INST(uint8_t, RMX_NHWC, false)

template <typename T>
static KernelFn pick_layout(int layout, bool norm) {
    if (layout == RMX_NCHW) return norm ? (KernelFn)rmx_cmn_kernel<T, RMX_NCHW, true> : (KernelFn)rmx_cmn_kernel<T, RMX_NCHW, false>;
    return norm ? (KernelFn)rmx_cmn_kernel<T, RMX_NHWC, true> : (KernelFn)rmx_cmn_kernel<T, RMX_NHWC, false>;
}

KernelFn select_cmn_kernel(int dtype, int layout, bool norm, const char **name) {
    static const char *names[3] = {"rmx_cmn_kernel<float", "rmx_cmn_kernel<__half", "rmx_cmn_kernel<unsigned char"};
    *name = names[dtype];
    switch (dtype) {
        case RMX_FP32: return pick_layout<float>(layout, norm);
        case RMX_FP16: return pick_layout<__half>(layout, norm);
        default: return pick_layout<uint8_t>(layout, norm);
    }
}

}  // namespace rmx
