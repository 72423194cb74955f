// Streaming neighbours of the colour family on packed RGB, one pass (3 bytes in per source, 3*sizeof(T) out):
//   table : out = lut[x]                     (Gamma: a 256-byte table per sample, built on the host)
//   blend : out = fma(a - b, ratio, b)       (Blend: two source batches of the same shape, the first one's ROI)
// Same wavefront -> (sample, strip of rows) mapping, realigned 16-byte loads and packed stores as the colour kernel.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

enum { POINT_TABLE = 0, POINT_BLEND = 1 };

// 8 packed RGB pixels -> v[c][k] = (float)lut[byte]: the byte is extracted once and indexes the wavefront's table in LDS
RMX_DEV void unpack8_table(const uint32_t (&w)[6], const uint8_t *lut, float (&v)[3][PX]) {
#pragma unroll
    for (int e = 0; e < 3 * PX; e++) {
        const uint32_t byte = (w[e >> 2] >> (8 * (e & 3))) & 0xffu;
        v[e % 3][e / 3] = (float)lut[byte];
    }
}

// MODE: 0 the general form; 1 whole 8-pixel groups and 16-byte aligned destination rows; 2 rows of 8 pixels and more at any
// alignment: the pipeline of 1, the short last group of a row moved left until it is whole (it recomputes up to seven pixels of
// its neighbour and stores the same values to the same places), groups stored at the element's own alignment.
template <typename T, int LAYOUT, int KIND, int MODE>
__global__ void __launch_bounds__(256) rmx_point_kernel(RmxKArgs a) {
    constexpr bool FAST = MODE != 0;
    constexpr bool ANY = MODE == 2;
    __shared__ uint32_t lut_words[4][64];  // one 256-byte table per wavefront of the workgroup
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    // fp32 and interleaved fp16 outputs: the lanes of a row exchange their runs through LDS before storing (store_packed_coalesced)
    constexpr bool COALESCE = MODE == 1 && coalesce_pays<T, LAYOUT>();
    uint32_t *slab = nullptr;
    if constexpr (COALESCE) {
        __shared__ __attribute__((aligned(16))) uint32_t slabs[4 * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>()];
        slab = slabs + (threadIdx.x / RMX_WAVE) * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>();
    }
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (uint32_t)a.wpb + (uint32_t)wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, strip;
    // workgroups in launch order (no XCD renumbering): the whole device walks the batch as one contiguous address stream,
    // and dealing the samples would only break that stream up (measured: 11-16 % slower)
    wave_to_sample(a, wave, s, strip, false);
    const RmxSample P = a.table[s];
    const int w = P.dst_w, h = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= h) return;
    const int r1 = min(r0 + srows, h);
    const int x1 = P.src_x, y1 = P.src_y;
    const float ratio = P.color[0];

    const uint8_t *lut = reinterpret_cast<const uint8_t *>(lut_words[wib]);
    if constexpr (KIND == POINT_TABLE) {
        lut_words[wib][lane] = reinterpret_cast<const uint32_t *>(a.extra)[(size_t)s * 64 + lane];
        wave_sync();
    }

    uint32_t row_stride32;
    const uint8_t *simg = sample_base(a, s, row_stride32);
    const size_t row_stride = row_stride32;
    const uint8_t *buf_end = a.src + a.src_bytes;
    // the second source has the first one's shape: same sample offset, same row stride, same extent
    const uint8_t *simg2 = (KIND == POINT_BLEND) ? a.src2 + (simg - a.src) : nullptr;
    const uint8_t *buf_end2 = (KIND == POINT_BLEND) ? a.src2 + a.src_bytes : nullptr;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    auto finish = [&](const uint32_t (&wa)[6], const uint32_t (&wb)[6], float (&v)[3][PX]) {
        if constexpr (KIND == POINT_TABLE) {
            unpack8_table(wa, lut, v);
        } else {
            float u[3][PX];
            unpack8(wa, v);
            unpack8(wb, u);
#pragma unroll
            for (int k = 0; k < PX; k++)
#pragma unroll
                for (int c = 0; c < 3; c++) v[c][k] = __builtin_fmaf(v[c][k] - u[c][k], ratio, u[c][k]);
        }
    };

    for (int xt = 0; xt < w; xt += RMX_WAVE * PX) {
        const int tw = min(w - xt, RMX_WAVE * PX);
        const int L = (tw + PX - 1) / PX;
        const int G = RMX_WAVE / L;
        const int lr = lane / L;
        const int g = lane - lr * L;
        int gx = xt + g * PX;
        if constexpr (ANY) gx = min(gx, w - PX);  // (the host admits this form for rows of 8 pixels and more)
        const int cnt = min(PX, w - gx);
        if constexpr (FAST) {
            // whole groups and aligned destination rows: the loads of NI row steps go out together, the stores follow
            constexpr int NI = 2;
            for (int rb = r0 + lr; rb < r1 && lr < G; rb += NI * G) {
                uint32_t wa[NI][6], wb[NI][6];
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int r = min(rb + i * G, r1 - 1);
                    const size_t off = (size_t)(y1 + r) * row_stride + (size_t)(x1 + gx) * 3;
                    load_realigned<7>(simg + off, buf_end, wa[i]);
                    if constexpr (KIND == POINT_BLEND) load_realigned<7>(simg2 + off, buf_end2, wb[i]);
                }
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int r = rb + i * G;
                    if (r < r1) {
                        float v[3][PX];
                        finish(wa[i], wb[i], v);
                        PackedGroup<T> packed;
                        pack_group_dir<T, LAYOUT, false>(v, packed);
                        if constexpr (COALESCE) store_packed_coalesced<T, LAYOUT>(slab, lane - g, g, L, dimg, a.dst_h, a.dst_w, r, gx, packed);
                        else store_packed<T, LAYOUT, sizeof(T) == 1, ANY>(dimg, a.dst_h, a.dst_w, r, gx, packed);
                    }
                }
            }
        } else {
            for (int r = r0 + lr; r < r1 && lr < G; r += G) {
                const size_t off = (size_t)(y1 + r) * row_stride + (size_t)(x1 + gx) * 3;
                uint32_t wa[6], wb[6];
                load_realigned<7>(simg + off, buf_end, wa);
                if constexpr (KIND == POINT_BLEND) load_realigned<7>(simg2 + off, buf_end2, wb);
                float v[3][PX];
                finish(wa, wb, v);
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, gx, cnt, v, false);
            }
        }
    }
}

template <int KIND, int MODE>
static KernelFn pick_point(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_point_kernel<float, RMX_NCHW, KIND, MODE>;
            case RMX_FP16: return (KernelFn)rmx_point_kernel<__half, RMX_NCHW, KIND, MODE>;
            default: return (KernelFn)rmx_point_kernel<uint8_t, RMX_NCHW, KIND, MODE>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_point_kernel<float, RMX_NHWC, KIND, MODE>;
        case RMX_FP16: return (KernelFn)rmx_point_kernel<__half, RMX_NHWC, KIND, MODE>;
        default: return (KernelFn)rmx_point_kernel<uint8_t, RMX_NHWC, KIND, MODE>;
    }
}

template <int KIND>
static KernelFn pick_point_mode(int mode, int dtype, int layout) {
    return mode == 1 ? pick_point<KIND, 1>(dtype, layout) : (mode == 2 ? pick_point<KIND, 2>(dtype, layout) : pick_point<KIND, 0>(dtype, layout));
}

KernelFn select_point_kernel(int kind, int dtype, int layout, int mode, const char **name) {
    *name = "rmx_point_kernel";
    return kind == POINT_BLEND ? pick_point_mode<POINT_BLEND>(mode, dtype, layout) : pick_point_mode<POINT_TABLE>(mode, dtype, layout);
}

}  // namespace rmx
