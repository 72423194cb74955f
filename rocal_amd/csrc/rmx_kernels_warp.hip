// K4: inverse-map affine warp (WarpAffine / Rotate), bilinear or nearest, constant-0 outside
// the source ROI; u8 NHWC in, T/LAYOUT out.
//
// A wavefront owns one 32x16 destination tile. The tile's corners are pushed through the
// affine map to get the source bounding box, which is staged into the wave's private LDS slice
// (dword per pixel, dword-aligned 128-bit global loads) and then gathered from LDS: source
// pixels that several destination pixels touch are fetched from HBM/L2 once per tile. When
// the box does not fit the slice (strong minification) the wave gathers from global memory.
// Each lane produces 8 adjacent destination pixels of one row and writes them with wide stores.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

extern __shared__ uint32_t rmx_lds_warp[];

constexpr int WTW = 32, WTH = 16;  // destination tile: 4 lanes x 8 px wide, 16 rows

RMX_DEV uint32_t load_px_global(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
}

template <typename T, int LAYOUT, bool NEAREST>
__global__ void __launch_bounds__(256) rmx_warp_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, gridDim.x) * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    const int s = (int)(wave / (uint32_t)a.strips);
    const int tile = (int)(wave % (uint32_t)a.strips);
    const int tiles_x = a.aux0;
    const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
    const RmxSample &P = a.table[s];
    const int dw = P.dst_w, dh = P.dst_h;
    const int X0 = tx * WTW, Y0 = ty * WTH;
    if (X0 >= dw || Y0 >= dh) return;

    const int xlo = P.src_x, ylo = P.src_y;
    const int xhi = xlo + P.src_w - 1, yhi = ylo + P.src_h - 1;
    const float m0 = P.m[0], m1 = P.m[1], m2 = P.m[2], m3 = P.m[3], m4 = P.m[4], m5 = P.m[5];
    const float dcx = (float)(dw >> 1), dcy = (float)(dh >> 1);
    const float scx = (float)(xlo + (P.src_w >> 1)), scy = (float)(ylo + (P.src_h >> 1));

    const size_t row_stride = (size_t)a.src_w * 3;
    const uint8_t *simg = a.src + (size_t)s * a.src_h * row_stride;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *lds = rmx_lds_warp + (size_t)wib * (a.lds_bytes >> 2);

    // source bounding box of the tile (wave-uniform), one pixel of margin, clipped to the ROI
    const int X1 = min(X0 + WTW, dw) - 1, Y1 = min(Y0 + WTH, dh) - 1;
    float bxmin = 3.0e38f, bxmax = -3.0e38f, bymin = 3.0e38f, bymax = -3.0e38f;
#pragma unroll
    for (int cy = 0; cy < 2; cy++)
#pragma unroll
        for (int cx = 0; cx < 2; cx++) {
            float xr = (float)(cx ? X1 : X0) - dcx, yr = (float)(cy ? Y1 : Y0) - dcy;
            float sx = __builtin_fmaf(xr, m0, __builtin_fmaf(yr, m1, m2)) + scx;
            float sy = __builtin_fmaf(xr, m3, __builtin_fmaf(yr, m4, m5)) + scy;
            bxmin = __builtin_fminf(bxmin, sx); bxmax = __builtin_fmaxf(bxmax, sx);
            bymin = __builtin_fminf(bymin, sy); bymax = __builtin_fmaxf(bymax, sy);
        }
    // keep the float->int conversions in range for degenerate matrices
    bxmin = __builtin_fmaxf(bxmin, -1.0e6f); bxmax = __builtin_fminf(bxmax, 1.0e6f);
    bymin = __builtin_fmaxf(bymin, -1.0e6f); bymax = __builtin_fminf(bymax, 1.0e6f);
    const int bx0 = max((int)floorf(bxmin) - 1, xlo), bx1 = min((int)floorf(bxmax) + 2, xhi);
    const int by0 = max((int)floorf(bymin) - 1, ylo), by1 = min((int)floorf(bymax) + 2, yhi);
    const int bw = bx1 - bx0 + 1, bh = by1 - by0 + 1;
    const bool empty = bw <= 0 || bh <= 0;
    const int items = (max(bw, 0) + 3) >> 2;
    const int pitch = items * 4;
    const bool use_lds = !empty && (size_t)bh * pitch * 4 <= (size_t)a.lds_bytes;

    if (use_lds) {
        int q = 0, j = lane;
        while (j >= items) { j -= items; q++; }
        while (q < bh) {
            const uint8_t *p = simg + (size_t)(by0 + q) * row_stride + (size_t)(bx0 + 4 * j) * 3;
            uint32_t w[3];
            load_realigned<4>(p, buf_end, w);
            uint4 px;
            px.x = w[0];
            px.y = __builtin_amdgcn_alignbyte(w[1], w[0], 3);
            px.z = __builtin_amdgcn_alignbyte(w[2], w[1], 2);
            px.w = w[2] >> 8;
            *reinterpret_cast<uint4 *>(lds + q * pitch + 4 * j) = px;
            j += RMX_WAVE;
            while (j >= items) { j -= items; q++; }
        }
        wave_sync();
    }

    const int lr = lane >> 2, g = lane & 3;
    const int y = Y0 + lr, x0 = X0 + g * PX;
    const int cnt = min(PX, dw - x0);
    if (y >= dh || cnt <= 0) return;
    const float yr = (float)y - dcy;
    float v[3][PX];
#pragma unroll
    for (int k = 0; k < PX; k++) {
        const float xr = (float)(x0 + k) - dcx;
        const float sx = __builtin_fmaf(xr, m0, __builtin_fmaf(yr, m1, m2)) + scx;
        const float sy = __builtin_fmaf(xr, m3, __builtin_fmaf(yr, m4, m5)) + scy;
        float fx, fy;
        if constexpr (NEAREST) {
            fx = floorf(sx + 0.5f);
            fy = floorf(sy + 0.5f);
        } else {
            fx = floorf(sx);
            fy = floorf(sy);
        }
        const bool oob = empty || fx < (float)xlo || fy < (float)ylo || fx > (float)xhi || fy > (float)yhi || !(fx == fx) || !(fy == fy);
        float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f;
        if (!oob) {
            const int ix0 = (int)fx, iy0 = (int)fy;
            const int ix1 = min(ix0 + 1, xhi), iy1 = min(iy0 + 1, yhi);
            uint32_t tl, tr, bl, br;
            if (use_lds) {
                const int cx0 = min(max(ix0 - bx0, 0), bw - 1), cx1 = min(max(ix1 - bx0, 0), bw - 1);
                const int cy0 = min(max(iy0 - by0, 0), bh - 1), cy1 = min(max(iy1 - by0, 0), bh - 1);
                // one multiply for the four taps: the right / lower neighbour is 0 or 1 column / row away
                const uint32_t *t0p = lds + __mul24(cy0, pitch) + cx0;
                const int dx = cx1 - cx0, dy = (cy1 - cy0) ? pitch : 0;
                tl = t0p[0];
                if constexpr (!NEAREST) {
                    tr = t0p[dx];
                    bl = t0p[dy];
                    br = t0p[dy + dx];
                }
            } else {
                tl = load_px_global(simg + (size_t)iy0 * row_stride + (size_t)ix0 * 3);
                if constexpr (!NEAREST) {
                    tr = load_px_global(simg + (size_t)iy0 * row_stride + (size_t)ix1 * 3);
                    bl = load_px_global(simg + (size_t)iy1 * row_stride + (size_t)ix0 * 3);
                    br = load_px_global(simg + (size_t)iy1 * row_stride + (size_t)ix1 * 3);
                }
            }
            if constexpr (NEAREST) {
                o0 = ubyte0(tl); o1 = ubyte1(tl); o2 = ubyte2(tl);
            } else {
                const float wx = sx - fx, wy = sy - fy;
                const float omx = 1.0f - wx, omy = 1.0f - wy;
                const float w00 = omy * omx, w01 = omy * wx, w10 = wy * omx;
                o0 = __builtin_fmaf(ubyte0(tl), w00, __builtin_fmaf(ubyte0(tr), w01, __builtin_fmaf(ubyte0(bl), w10, ubyte0(br) * wy * wx)));
                o1 = __builtin_fmaf(ubyte1(tl), w00, __builtin_fmaf(ubyte1(tr), w01, __builtin_fmaf(ubyte1(bl), w10, ubyte1(br) * wy * wx)));
                o2 = __builtin_fmaf(ubyte2(tl), w00, __builtin_fmaf(ubyte2(tr), w01, __builtin_fmaf(ubyte2(bl), w10, ubyte2(br) * wy * wx)));
            }
        }
        v[0][k] = o0; v[1][k] = o1; v[2][k] = o2;
    }
    // whole group into 16-byte aligned destination rows: packed stores (a.aux1 is set by the host when every
    // written width and the padded width are multiples of 8 and the destination base is 16-byte aligned)
    if (a.aux1 && cnt == PX) {
        PackedGroup<T> packed;
        pack_group_dir<T, LAYOUT, false>(v, packed);
        store_packed<T, LAYOUT>(dimg, a.dst_h, a.dst_w, y, x0, packed);
    } else {
        store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, y, x0, cnt, v, false);
    }
}

template <bool NEAREST>
static KernelFn pick(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_warp_kernel<float, RMX_NCHW, NEAREST>;
            case RMX_FP16: return (KernelFn)rmx_warp_kernel<__half, RMX_NCHW, NEAREST>;
            default: return (KernelFn)rmx_warp_kernel<uint8_t, RMX_NCHW, NEAREST>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_warp_kernel<float, RMX_NHWC, NEAREST>;
        case RMX_FP16: return (KernelFn)rmx_warp_kernel<__half, RMX_NHWC, NEAREST>;
        default: return (KernelFn)rmx_warp_kernel<uint8_t, RMX_NHWC, NEAREST>;
    }
}

KernelFn select_warp_kernel(int interp, int dtype, int layout, const char **name) {
    *name = "rmx_warp_kernel";
    return interp == RMX_INTERP_NEAREST ? pick<true>(dtype, layout) : pick<false>(dtype, layout);
}

}  // namespace rmx
