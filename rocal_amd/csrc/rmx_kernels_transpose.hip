// Transpose of the image axes (height <-> width) of every sample's window, channels kept last (output [N, W, H, C]) or moved
// to the front (output [N, C, W, H]); the two permutations of rocAL's Transpose node that move pixels
// (geometry_augmentations/node_transpose.cpp:52-66: {1,0,2} and {2,1,0}); the other two it allows on images, {0,1,2} and
// {2,0,1}, are layout changes of the streaming kernel.
// One wavefront = a 32 x 32 pixel tile: rows are read as 8-pixel groups (realigned 16-byte loads), parked in the wavefront's LDS
// slice as one dword per pixel (row pitch 33: the transposed reads fall on different banks) and written out as 8-pixel groups
// of the transposed rows.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

constexpr int TT = 32;          // tile edge in pixels
constexpr int TPITCH = TT + 1;  // LDS row pitch in dwords

template <typename T, int LAYOUT>
__global__ void __launch_bounds__(256) rmx_transpose_kernel(RmxKArgs a) {
    __shared__ uint32_t tiles[4][TT * TPITCH];
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, tile;
    wave_to_sample(a, wave, s, tile, false);  // no XCD renumbering in this kernel: batch order keeps the address stream contiguous
    const RmxSample &P = a.table[s];
    const int w = P.src_w, h = P.src_h;  // the window; the output is h columns wide and w rows high
    const int ty = tile / a.aux0, tx = tile - ty * a.aux0;
    const int y0 = ty * TT, x0 = tx * TT;
    if (y0 >= h || x0 >= w) return;
    uint32_t row_stride;
    const uint8_t *simg = sample_base(a, s, row_stride);
    const uint8_t *buf_end = a.src + a.src_bytes;
    uint32_t *lds = tiles[wib];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int gi = lane + RMX_WAVE * j;
        const int r = gi >> 2, g = gi & 3;
        const int sy = y0 + r, sx = x0 + PX * g;
        if (sy < h && sx < w) {
            const int cnt = min(PX, w - sx);
            uint32_t d[6];
            load_realigned<7>(simg + (size_t)(P.src_y + sy) * row_stride + (size_t)(P.src_x + sx) * 3, buf_end, d);
#pragma unroll
            for (int k = 0; k < PX; k++) {
                if (k < cnt) {
                    uint32_t px = 0;
#pragma unroll
                    for (int c = 0; c < 3; c++) {
                        const int byte = 3 * k + c;
                        px |= ((d[byte >> 2] >> (8 * (byte & 3))) & 0xffu) << (8 * c);
                    }
                    lds[r * TPITCH + PX * g + k] = px;
                }
            }
        }
    }
    wave_sync();
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int gi = lane + RMX_WAVE * j;
        const int c = gi >> 2, g = gi & 3;  // source column = output row; 8 source rows = 8 output columns
        const int oy = x0 + c, ox = y0 + PX * g;
        if (oy < w && ox < h) {
            const int cnt = min(PX, h - ox);
            float v[3][PX];
#pragma unroll
            for (int k = 0; k < PX; k++) {
                const uint32_t px = lds[(PX * g + min(k, cnt - 1)) * TPITCH + c];
                v[0][k] = ubyte0(px);
                v[1][k] = ubyte1(px);
                v[2][k] = ubyte2(px);
            }
            store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, oy, ox, cnt, v, false);
        }
    }
}

template <typename T>
static KernelFn pick(int layout) {
    return layout == RMX_NCHW ? (KernelFn)rmx_transpose_kernel<T, RMX_NCHW> : (KernelFn)rmx_transpose_kernel<T, RMX_NHWC>;
}

KernelFn select_transpose_kernel(int dtype, int layout, const char **name) {
    *name = "rmx_transpose_kernel";
    switch (dtype) {
        case RMX_FP32: return pick<float>(layout);
        case RMX_FP16: return pick<__half>(layout);
        default: return pick<uint8_t>(layout);
    }
}

}  // namespace rmx
