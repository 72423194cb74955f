// K3: per-pixel colour ops on packed RGB, one streaming pass (3 bytes in, 3*sizeof(T) out).
//   linear : out = fma(x - p2, p0, p1)   (Brightness: p0=alpha,p1=beta,p2=0; Contrast: p0=factor,p1=p2=center)
//   twist  : RGB->HSV on the 0..255 scale, hue shift (sextants), saturation scale, HSV->RGB,
//            then fma(c, alpha, beta)    (ColorTwist; Hue and Saturation are twists with fixed alpha/beta)
// The two reciprocals of the HSV path (1/delta, 1/cmax) have integer arguments in 1..255 and
// come from a 256-entry LDS table of correctly rounded reciprocals, so the result is
// bit-identical to IEEE division by the same integers without paying for a division per pixel.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

enum { COLOR_LINEAR = 0, COLOR_TWIST = 1 };


// HSV -> RGB per hue sector: each output channel is one of V, q = V - V*S*f, p = V - V*S, t = p + V*S*f. All four have the form
// fma(sg, V*S*f, fma(nb, V*S, V)) with sg in {0,-1,+1} and nb in {0,-1}: a multiplication by 0 or +-1 is exact, so the two FMAs
// round exactly where the subtraction and the addition of the plain formulas round. The six coefficients of a sector come from
// a small LDS table indexed by the sector, which replaces the compare/select network (14 compares and selects per pixel).
//   sector:  0 1 2 3 4 5      r: V q p p t V      g: t V V q p p      b: p p t V V q
struct SectorRow {
    float sg[3], nb0;  // sg of r,g,b ; nb of r
    float nb1, nb2, pad0, pad1;  // nb of g,b
};
RMX_DEV void sector_row(int hi, SectorRow &row) {
    // codes: 0 = V, 1 = q, 2 = p, 3 = t
    const int rc[6] = {0, 1, 2, 2, 3, 0}, gc[6] = {3, 0, 0, 1, 2, 2}, bc[6] = {2, 2, 3, 0, 0, 1};
    const int h = hi == 6 ? 0 : (hi > 5 ? 5 : hi);  // row 6 repeats row 0 (see the hue reduction), row 7 is never read
    const int code[3] = {rc[h], gc[h], bc[h]};
    float sg[3], nb[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sg[c] = code[c] == 1 ? -1.0f : (code[c] == 3 ? 1.0f : 0.0f);
        nb[c] = code[c] >= 2 ? -1.0f : 0.0f;
    }
    row.sg[0] = sg[0]; row.sg[1] = sg[1]; row.sg[2] = sg[2]; row.nb0 = nb[0];
    row.nb1 = nb[1]; row.nb2 = nb[2]; row.pad0 = 0.0f; row.pad1 = 0.0f;
}

// Branch-free: lanes of a wavefront hold pixels of different hue sectors, so
// branches would run every case one after the other under changing execution masks.
RMX_DEV void twist_px(float &r, float &g, float &b, const float *rcp, const SectorRow *sect, float alpha, float beta, float shift, float shift2, float shift4, float satf) {
    const float cmax = __builtin_fmaxf(__builtin_fmaxf(r, g), b);
    const float cmin = __builtin_fminf(__builtin_fminf(r, g), b);
    const float delta = cmax - cmin;
    const float rd = rcp[(int)delta];      // 0 when delta == 0
    float s = delta * rcp[(int)cmax];
    // A grey pixel needs no case of its own: r == g == b makes it a "red is largest" pixel with g - b == 0.
    const bool is_r = cmax == r, is_g = cmax == g;
    const float num = is_r ? (g - b) : (is_g ? (b - r) : (r - g));
    // sextant offset 0 / 2 / 4 plus the hue shift, the three sums made once per sample
    const float add = is_r ? shift : (is_g ? shift2 : shift4);
    float hh = __builtin_fmaf(num, rd, add);
    // back into [0, 6]: one addition of +6, -6 or 0. A value just below zero can round to exactly 6.0 here; row 6 of the sector
    // table repeats row 0 and fract(6.0) is 0, which is the pixel a second reduction to 0.0 would give.
    hh = hh + (hh < 0.0f ? 6.0f : (hh >= 6.0f ? -6.0f : 0.0f));
    s = s * satf;
    s = __builtin_fminf(__builtin_fmaxf(s, 0.0f), 1.0f);
    // sector and fraction; hh lies in [0, 6], where hh - floor(hh) is exact and equals hh - trunc(hh)
    const SectorRow row = sect[(int)hh];
    const float hf = __builtin_amdgcn_fractf(hh);
    const float vsat = cmax * s;
    const float vsatf = vsat * hf;
    const float ro = __builtin_fmaf(row.sg[0], vsatf, __builtin_fmaf(row.nb0, vsat, cmax));
    const float go = __builtin_fmaf(row.sg[1], vsatf, __builtin_fmaf(row.nb1, vsat, cmax));
    const float bo = __builtin_fmaf(row.sg[2], vsatf, __builtin_fmaf(row.nb2, vsat, cmax));
    r = __builtin_fmaf(ro, alpha, beta);
    g = __builtin_fmaf(go, alpha, beta);
    b = __builtin_fmaf(bo, alpha, beta);
}

template <typename T, int LAYOUT, int KIND, bool FAST>
__global__ void __launch_bounds__(256) rmx_color_kernel(RmxKArgs a) {
    __shared__ float rcp[256];
    __shared__ __attribute__((aligned(16))) SectorRow sect[8];
    if constexpr (KIND == COLOR_TWIST) {
        int t = threadIdx.x;
        if (t < 256) rcp[t] = (t == 0) ? 0.0f : 1.0f / (float)t;
        if (t < 8) sector_row(t, sect[t]);
        __syncthreads();
    }
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (uint32_t)a.wpb + (threadIdx.x / RMX_WAVE);
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    const int s = (int)(wave / (uint32_t)a.strips);
    const int strip = (int)(wave % (uint32_t)a.strips);
    // whole table row in one round trip (the empty statement keeps the fetch above the early exit)
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.flags), "s"(P.color[0]), "s"(P.color[3]));
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
    auto colour = [&](float (&v)[3][PX]) {
#pragma unroll
        for (int k = 0; k < PX; k++) {
            if constexpr (KIND == COLOR_TWIST) {
                twist_px(v[0][k], v[1][k], v[2][k], rcp, sect, p0, p1, sh0, sh2, sh4, p3);
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
        const int gx = xt + g * PX;
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
                        store_packed<T, LAYOUT, sizeof(T) == 1>(dimg, a.dst_h, a.dst_w, r, gx, packed);  // u8: streaming stores
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

template <int KIND, bool FAST>
static KernelFn pick(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NCHW, KIND, FAST>;
            case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NCHW, KIND, FAST>;
            default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NCHW, KIND, FAST>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NHWC, KIND, FAST>;
        case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NHWC, KIND, FAST>;
        default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NHWC, KIND, FAST>;
    }
}

KernelFn select_color_kernel(int kind, int dtype, int layout, bool fast, const char **name) {
    *name = "rmx_color_kernel";
    if (fast) return kind == COLOR_TWIST ? pick<COLOR_TWIST, true>(dtype, layout) : pick<COLOR_LINEAR, true>(dtype, layout);
    return kind == COLOR_TWIST ? pick<COLOR_TWIST, false>(dtype, layout) : pick<COLOR_LINEAR, false>(dtype, layout);
}

}  // namespace rmx
