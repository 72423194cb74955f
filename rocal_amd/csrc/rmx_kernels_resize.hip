// K2: ROI crop -> bilinear (or nearest) resize -> [u8 quantise] -> [mirror] -> [normalise]
//     -> layout transpose -> cast, in one pass. Serves Resize / CropResize / ROIResize /
//     ResizeCropMirror / ResizeMirrorNormalize and the fused RandomResizedCrop + CMN chain.
//
// Scheduling is wavefront-granular: every wavefront owns a strip of output rows of one sample
// and a private slice of LDS; there is no workgroup barrier anywhere. Per step the wave
//   1. stages the source rows its G output rows touch into LDS with dword-aligned 128-bit
//      global loads (12 useful bytes = 4 packed pixels per lane), expanding each pixel to one
//      dword so that the gather below is bank-friendly and needs no byte addressing,
//   2. gathers the 2x2 neighbourhoods from LDS (two adjacent-dword reads per pixel), blends
//      in fp32 in the reference's FMA order, applies the epilogue and
//   3. writes 8 pixels per lane with 128-bit stores (fp16 planar).
// HBM-bound: each source byte of the window is fetched once per strip (halo rows hit L1/L2).
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

extern __shared__ uint32_t rmx_lds[];

// source coordinate of resized index u (rocal bilinear law: u*ratio + (ratio-1)/2 + roi.lo)
RMX_DEV float src_coord(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}

template <typename T, int LAYOUT, bool NORM, bool QUANT, bool NEAREST>
__global__ void __launch_bounds__(256) rmx_resize_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, gridDim.x) * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    const int s = (int)(wave / (uint32_t)a.strips);
    const int strip = (int)(wave % (uint32_t)a.strips);
    const RmxSample &P = a.table[s];

    const int dw = P.dst_w, dh = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= dh || dw <= 0) return;
    const int r1 = min(r0 + srows, dh);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;

    const int xlo = P.src_x, ylo = P.src_y;
    const int xhi = xlo + P.src_w - 1, yhi = ylo + P.src_h - 1;
    const float rx = P.rx, ry = P.ry;
    const float offx = (rx - 1.0f) * 0.5f, offy = (ry - 1.0f) * 0.5f;
    const float fxlo = (float)xlo, fylo = (float)ylo;
    const int pcx = P.pc_x, pcy = P.pc_y;

    const size_t row_stride = (size_t)a.src_w * 3;
    const uint8_t *simg = a.src + (size_t)s * a.src_h * row_stride;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *lds = rmx_lds + (size_t)wib * (a.lds_bytes >> 2);

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    const int tile_w = a.aux1;  // output columns per x-tile (multiple of PX, <= 64*PX)
    for (int xt = 0; xt < dw; xt += tile_w) {
        const int tw = min(dw - xt, tile_w);
        const int L = (tw + PX - 1) / PX;
        const int G = RMX_WAVE / L;
        const int lr = lane / L;
        const int g = lane - lr * L;
        const int t0 = xt + g * PX;                 // first window-relative column of the group
        const int cnt = min(PX, dw - t0);
        const bool lane_on = lr < G;

        // tile-wide source column range (wave-uniform)
        const int u_first = pcx + xt, u_last = pcx + xt + tw - 1;
        const int ixmin = (int)floorf(src_coord(u_first, rx, offx, fxlo));
        const int ixmax = (int)floorf(src_coord(u_last, rx, offx, fxlo));
        const int cs = max(min(ixmin, xhi), xlo);
        const int ce = max(min(ixmax + 1, xhi), xlo);
        const int nc = ce - cs + 1;
        const int items = (nc + 3) >> 2;
        const int pitch = 4 + items * 4 + 4;
        const bool rep_l = ixmin < xlo, rep_r = ixmax + 1 > xhi;

        // per-lane column taps, fixed for the whole strip
        int off[PX];
        float wx[PX];
#pragma unroll
        for (int k = 0; k < PX; k++) {
            int u = pcx + min(t0 + k, dw - 1);
            float sx = src_coord(u, rx, offx, fxlo);
            float fx = floorf(sx);
            wx[k] = sx - fx;
            off[k] = 4 + ((int)fx - cs);
        }

        for (int rs = r0; rs < r1; rs += G) {
            // rows of this step: rs .. min(rs+G, r1)-1 ; virtual source rows they touch
            const int re = min(rs + G, r1) - 1;
            const int iy_first = (int)floorf(src_coord(pcy + rs, ry, offy, fylo));
            const int iy_last = (int)floorf(src_coord(pcy + re, ry, offy, fylo));
            const int nrows = iy_last - iy_first + 2;

            // ---- stage: (row slot q, item j) pairs dealt over the lanes
            {
                int q = 0, j = lane;
                while (j >= items) { j -= items; q++; }
                while (q < nrows) {
                    const int ysrc = max(min(iy_first + q, yhi), ylo);
                    const uint8_t *p = simg + (size_t)ysrc * row_stride + (size_t)(cs + 4 * j) * 3;
                    uint32_t w[3];
                    load_realigned<4>(p, buf_end, w);
                    uint4 px;
                    px.x = w[0];
                    px.y = __builtin_amdgcn_alignbyte(w[1], w[0], 3);
                    px.z = __builtin_amdgcn_alignbyte(w[2], w[1], 2);
                    px.w = w[2] >> 8;
                    *reinterpret_cast<uint4 *>(lds + q * pitch + 4 + 4 * j) = px;
                    j += RMX_WAVE;
                    while (j >= items) { j -= items; q++; }
                }
            }
            wave_sync();
            if (rep_l || rep_r) {
                if (lane < nrows) {
                    uint32_t *row = lds + lane * pitch;
                    if (rep_l) row[3] = row[4];
                    if (rep_r) row[4 + nc] = row[4 + nc - 1];
                }
                wave_sync();
            }

            // ---- gather + blend + epilogue
            const int r = rs + lr;
            if (lane_on && r <= re && cnt > 0) {
                float sy = src_coord(pcy + r, ry, offy, fylo);
                float fy = floorf(sy);
                float wy = sy - fy;
                const uint32_t *row0 = lds + ((int)fy - iy_first) * pitch;
                const uint32_t *row1 = row0 + pitch;
                float v[3][PX];
                if constexpr (NEAREST) {
                    const uint32_t *rsel = wy < 0.5f ? row0 : row1;
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        uint32_t p = rsel[off[k] + (wx[k] < 0.5f ? 0 : 1)];
                        v[0][k] = ubyte0(p);
                        v[1][k] = ubyte1(p);
                        v[2][k] = ubyte2(p);
                    }
                } else {
                    const float omy = 1.0f - wy;
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        uint32_t tl = row0[off[k]], tr = row0[off[k] + 1];
                        uint32_t bl = row1[off[k]], br = row1[off[k] + 1];
                        float omx = 1.0f - wx[k];
                        float w00 = omy * omx, w01 = omy * wx[k], w10 = wy * omx;
                        v[0][k] = __builtin_fmaf(ubyte0(tl), w00, __builtin_fmaf(ubyte0(tr), w01, __builtin_fmaf(ubyte0(bl), w10, ubyte0(br) * wy * wx[k])));
                        v[1][k] = __builtin_fmaf(ubyte1(tl), w00, __builtin_fmaf(ubyte1(tr), w01, __builtin_fmaf(ubyte1(bl), w10, ubyte1(br) * wy * wx[k])));
                        v[2][k] = __builtin_fmaf(ubyte2(tl), w00, __builtin_fmaf(ubyte2(tr), w01, __builtin_fmaf(ubyte2(bl), w10, ubyte2(br) * wy * wx[k])));
                    }
                }
#pragma unroll
                for (int c = 0; c < 3; c++)
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        float t = v[c][k];
                        if constexpr (QUANT) t = round_u8(t);
                        if constexpr (NORM) t = __builtin_fmaf(t, sc[c], bi[c]);
                        v[c][k] = t;
                    }
                const int x0 = hf ? (dw - t0 - cnt) : t0;
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, x0, cnt, v, hf);
            }
            wave_sync();  // next step overwrites the LDS rows just read
        }
    }
}

template <typename T, int LAYOUT, bool NEAREST>
static KernelFn pick3(bool norm, bool quant) {
    if (norm && quant) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, true, NEAREST>;
    if (norm) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, false, NEAREST>;
    return (KernelFn)rmx_resize_kernel<T, LAYOUT, false, false, NEAREST>;
}

template <bool NEAREST>
static KernelFn pick(int dtype, int layout, bool norm, bool quant) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return pick3<float, RMX_NCHW, NEAREST>(norm, quant);
            case RMX_FP16: return pick3<__half, RMX_NCHW, NEAREST>(norm, quant);
            default: return pick3<uint8_t, RMX_NCHW, NEAREST>(norm, quant);
        }
    }
    switch (dtype) {
        case RMX_FP32: return pick3<float, RMX_NHWC, NEAREST>(norm, quant);
        case RMX_FP16: return pick3<__half, RMX_NHWC, NEAREST>(norm, quant);
        default: return pick3<uint8_t, RMX_NHWC, NEAREST>(norm, quant);
    }
}

KernelFn select_resize_linear_kernel(int dtype, int layout, bool norm, bool quant, const char **name) {
    *name = "rmx_resize_kernel";
    return pick<false>(dtype, layout, norm, quant);
}

KernelFn select_resize_nearest_kernel(int dtype, int layout, bool norm, bool quant, const char **name) {
    *name = "rmx_resize_kernel";
    return pick<true>(dtype, layout, norm, quant);
}

}  // namespace rmx
