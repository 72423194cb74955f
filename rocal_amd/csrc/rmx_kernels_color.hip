// K3: per-pixel colour ops on packed RGB, one streaming pass (3 bytes in, 3*sizeof(T) out).
//   linear : out = fma(x - p2, p0, p1)   (Brightness: p0=alpha,p1=beta,p2=0; Contrast: p0=factor,p1=p2=center)
//   twist  : RGB->HSV on the 0..255 scale, hue shift (sextants), saturation scale, HSV->RGB,
//            then fma(c, alpha, beta)    (ColorTwist; Hue and Saturation are twists with fixed alpha/beta)
// The two reciprocals of the HSV path (1/delta, 1/cmax) have integer arguments in 1..255 and
// come from a 256-entry LDS table of correctly rounded reciprocals, so the result is
// bit-identical to IEEE division by the same integers without paying for a division per pixel.
#include "rmx_device.h"
#include "rmx_color_math.h"
#include "rmx_launch.h"

namespace rmx {

// COLOR_TWIST1: the twist for batches in which no sample's hue shift lies within 2e-5 of one sextant (one comparison brings
// the hue back into range, see HueWrap)
enum { COLOR_LINEAR = 0, COLOR_TWIST = 1, COLOR_TWIST1 = 2 };


// MODE: 0 the general form; 1 whole 8-pixel groups and 16-byte aligned destination rows; 2 rows of 8 pixels and more at any
// alignment: the pipeline of 1, the short last group of a row moved left until it is whole (it recomputes up to seven pixels of
// its neighbour and stores the same values to the same places), groups stored at the element's own alignment.
template <typename T, int LAYOUT, int KIND_ARG, int MODE>
__global__ void __launch_bounds__(256) rmx_color_kernel(RmxKArgs a) {
    constexpr int KIND = KIND_ARG == COLOR_TWIST1 ? COLOR_TWIST : KIND_ARG;
    constexpr int WRAP = KIND_ARG == COLOR_TWIST1 ? HUE_WRAP_ONE : HUE_WRAP_BOTH;
    constexpr bool FAST = MODE != 0;
    constexpr bool ANY = MODE == 2;
    __shared__ ColorTables tabs;
    const float *rcp = tabs.rcp;
    const SectorRow *sect = tabs.sect;
    // The workgroup copies the two tables of the twist from device memory into LDS, 16 bytes per thread (two for the first
    // threads of a workgroup of one wavefront). The reads are started here and written to LDS behind the fetch of the table
    // row below, so that the two round trips overlap.
    constexpr unsigned TAB_PIECES = sizeof(ColorTables) / 16;
    uint4 tab0 = {}, tab1 = {};
    if constexpr (KIND == COLOR_TWIST) {
        const uint4 *rom = reinterpret_cast<const uint4 *>(&rmx_color_tables_rom);
        if (threadIdx.x < TAB_PIECES) tab0 = rom[threadIdx.x];
        if (threadIdx.x + blockDim.x < TAB_PIECES) tab1 = rom[threadIdx.x + blockDim.x];
    }
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    // fp32 and interleaved fp16 outputs: the lanes of a row exchange their runs through LDS before storing (store_packed_coalesced)
    constexpr bool COALESCE = MODE == 1 && coalesce_pays<T, LAYOUT>();
    uint32_t *slab = nullptr;
    if constexpr (COALESCE) {
        __shared__ __attribute__((aligned(16))) uint32_t slabs[4 * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>()];
        slab = slabs + (threadIdx.x / RMX_WAVE) * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>();
    }
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (uint32_t)a.wpb + (threadIdx.x / RMX_WAVE);
    wave = __builtin_amdgcn_readfirstlane(wave);
    int s, strip;
    // workgroups in launch order (no XCD renumbering): the whole device walks the batch as one contiguous address stream,
    // and dealing the samples would only break that stream up (measured: 11-16 % slower)
    // (a wavefront beyond the batch fetches the last wavefront's row: it stays for the workgroup's barrier and leaves then)
    wave_to_sample(a, min(wave, nwaves - 1), s, strip, false);
    // whole table row in one round trip (the empty statement keeps the fetch above the barrier and the early exit)
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.flags), "s"(P.color[0]), "s"(P.color[3]));
    if constexpr (KIND == COLOR_TWIST) {
        uint4 *ram = reinterpret_cast<uint4 *>(&tabs);
        if (threadIdx.x < TAB_PIECES) ram[threadIdx.x] = tab0;
        if (threadIdx.x + blockDim.x < TAB_PIECES) ram[threadIdx.x + blockDim.x] = tab1;
        __syncthreads();
    }
    if (wave >= nwaves) return;
    const int w = P.dst_w, h = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= h) return;
    const int r1 = min(r0 + srows, h);
    const int x1 = P.src_x, y1 = P.src_y;
    const float p0 = P.color[0], p1 = P.color[1], p2 = P.color[2], p3 = P.color[3];

    uint32_t row_stride32;
    const uint8_t *simg = sample_base(a, s, row_stride32);
    const size_t row_stride = row_stride32;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    // sextant offset 0 / 2 / 4 plus the hue shift, summed once per wavefront and kept in vector registers, so that the choice
    // between them is two selects per pixel (from scalar registers the compiler selects a constant and adds the shift again)
    float sh0 = p2, sh2 = p2 + 2.0f, sh4 = p2 + 4.0f;
    if constexpr (KIND == COLOR_TWIST) asm volatile("" : "+v"(sh0), "+v"(sh2), "+v"(sh4));
    const HueWrap hw = hue_wrap_of(p2);
    float wrap_t = hw.t, wrap_at = hw.at, wrap_af = hw.af;
    if constexpr (WRAP == HUE_WRAP_ONE) asm volatile("" : "+v"(wrap_t), "+v"(wrap_at), "+v"(wrap_af));
    auto colour = [&](float (&v)[3][PX]) {
#pragma unroll
        for (int k = 0; k < PX; k++) {
            if constexpr (KIND == COLOR_TWIST) {
                twist_px<WRAP>(v[0][k], v[1][k], v[2][k], rcp, sect, p0, p1, sh0, sh2, sh4, p3, wrap_t, wrap_at, wrap_af);
            } else {
#pragma unroll
                for (int c = 0; c < 3; c++) v[c][k] = __builtin_fmaf(v[c][k] - p2, p0, p1);
            }
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
            // whole groups and aligned destination rows: the loads of up to NI row steps go out together,
            // the stores follow (one memory round trip per strip, see the CropMirrorNormalize kernel)
            constexpr int NI = (KIND == COLOR_TWIST) ? 1 : 4;  // twist: one group per step keeps 65 registers (7 wavefronts per SIMD); two need 111
            for (int rb = r0 + lr; rb < r1 && lr < G; rb += NI * G) {
                const uint32_t *q[NI];
                uint32_t ph[NI];
                bool safe = true;
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int r = min(rb + i * G, r1 - 1);
                    const uint8_t *p = simg + (size_t)(y1 + r) * row_stride + (size_t)(x1 + gx) * 3;
                    ph[i] = (uint32_t)((uintptr_t)p & 3u);
                    q[i] = reinterpret_cast<const uint32_t *>(p - ph[i]);
                    safe = safe && ((const uint8_t *)(q[i] + 7) <= buf_end);
                }
                uint32_t wd[NI][6];
                if (safe) {
                    u32x4_a4 t[NI];
                    u32x3_a4 u[NI];
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        t[i] = *reinterpret_cast<const u32x4_a4 *>(q[i]);
                        u[i] = *reinterpret_cast<const u32x3_a4 *>(q[i] + 4);
                    }
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        const uint32_t d[7] = {t[i].x, t[i].y, t[i].z, t[i].w, u[i].x, u[i].y, u[i].z};
#pragma unroll
                        for (int j = 0; j < 6; j++) wd[i][j] = __builtin_amdgcn_alignbyte(d[j + 1], d[j], ph[i]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NI; i++)
                        load_realigned<7>(reinterpret_cast<const uint8_t *>(q[i]) + ph[i], buf_end, wd[i]);
                }
#pragma unroll
                for (int i = 0; i < NI; i++) {
                    const int r = rb + i * G;
                    if (r < r1) {
                        float v[3][PX];
                        unpack8(wd[i], v);
                        colour(v);
                        PackedGroup<T> packed;
                        pack_group_dir<T, LAYOUT, false>(v, packed);
                        if constexpr (COALESCE) store_packed_coalesced<T, LAYOUT>(slab, lane - g, g, L, dimg, a.dst_h, a.dst_w, r, gx, packed);
                        else store_packed<T, LAYOUT, sizeof(T) == 1, ANY>(dimg, a.dst_h, a.dst_w, r, gx, packed);  // u8: streaming stores
                    }
                }
            }
        } else {
            for (int r = r0 + lr; r < r1 && lr < G; r += G) {
                const uint8_t *p = simg + (size_t)(y1 + r) * row_stride + (size_t)(x1 + gx) * 3;
                uint32_t wd[6];
                load_realigned<7>(p, buf_end, wd);
                float v[3][PX];
                unpack8(wd, v);
                colour(v);
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, gx, cnt, v, false);
            }
        }
    }
}

template <int KIND, int MODE>
static KernelFn pick(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NCHW, KIND, MODE>;
            case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NCHW, KIND, MODE>;
            default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NCHW, KIND, MODE>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NHWC, KIND, MODE>;
        case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NHWC, KIND, MODE>;
        default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NHWC, KIND, MODE>;
    }
}

template <int KIND>
static KernelFn pick_mode(int mode, int dtype, int layout) {
    return mode == 1 ? pick<KIND, 1>(dtype, layout) : (mode == 2 ? pick<KIND, 2>(dtype, layout) : pick<KIND, 0>(dtype, layout));
}

// kind: 0 linear, 1 twist, 2 twist for batches whose hue shifts all allow the single comparison
KernelFn select_color_kernel(int kind, int dtype, int layout, int mode, const char **name) {
    *name = "rmx_color_kernel";
    if (kind == COLOR_TWIST1) return pick_mode<COLOR_TWIST1>(mode, dtype, layout);
    return kind == COLOR_TWIST ? pick_mode<COLOR_TWIST>(mode, dtype, layout) : pick_mode<COLOR_LINEAR>(mode, dtype, layout);
}

}  // namespace rmx
