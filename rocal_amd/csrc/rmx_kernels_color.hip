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

RMX_DEV void twist_px(float &r, float &g, float &b, const float *rcp, float alpha, float beta, float shift, float satf) {
    float cmax = __builtin_fmaxf(__builtin_fmaxf(r, g), b);
    float cmin = __builtin_fminf(__builtin_fminf(r, g), b);
    float delta = cmax - cmin;
    float rd = rcp[(int)delta];      // 0 when delta == 0
    float s = delta * rcp[(int)cmax];
    float num, add;
    if (cmax == r) {
        num = g - b;
        add = 0.0f;
    } else if (cmax == g) {
        num = b - r;
        add = 2.0f;
    } else {
        num = r - g;
        add = 4.0f;
    }
    if (delta == 0.0f) {
        num = 0.0f;
        add = 0.0f;
    }
    float hh = __builtin_fmaf(num, rd, add + shift);
    if (hh < 0.0f) hh += 6.0f;
    if (hh >= 6.0f) hh -= 6.0f;
    s = s * satf;
    s = __builtin_fminf(__builtin_fmaxf(s, 0.0f), 1.0f);
    int hi = (int)hh;
    float hf = hh - (float)hi;
    float vsat = cmax * s;
    float vsatf = vsat * hf;
    float pp = cmax - vsat;
    float qq = cmax - vsatf;
    float tt = pp + vsatf;
    float ro, go, bo;
    switch (hi) {
        case 0: ro = cmax; go = tt; bo = pp; break;
        case 1: ro = qq; go = cmax; bo = pp; break;
        case 2: ro = pp; go = cmax; bo = tt; break;
        case 3: ro = pp; go = qq; bo = cmax; break;
        case 4: ro = tt; go = pp; bo = cmax; break;
        default: ro = cmax; go = pp; bo = qq; break;
    }
    r = __builtin_fmaf(ro, alpha, beta);
    g = __builtin_fmaf(go, alpha, beta);
    b = __builtin_fmaf(bo, alpha, beta);
}

template <typename T, int LAYOUT, int KIND>
__global__ void __launch_bounds__(256) rmx_color_kernel(RmxKArgs a) {
    __shared__ float rcp[256];
    if constexpr (KIND == COLOR_TWIST) {
        int t = threadIdx.x;
        if (t < 256) rcp[t] = (t == 0) ? 0.0f : 1.0f / (float)t;
        __syncthreads();
    }
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = blockIdx.x * (blockDim.x / RMX_WAVE) + (threadIdx.x / RMX_WAVE);
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    const int s = (int)(wave / (uint32_t)a.strips);
    const int strip = (int)(wave % (uint32_t)a.strips);
    const RmxSample &P = a.table[s];
    const int w = P.dst_w, h = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= h) return;
    const int r1 = min(r0 + srows, h);
    const int x1 = P.src_x, y1 = P.src_y;
    const float p0 = P.color[0], p1 = P.color[1], p2 = P.color[2], p3 = P.color[3];

    const size_t row_stride = (size_t)a.src_w * 3;
    const uint8_t *simg = a.src + (size_t)s * a.src_h * row_stride;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    for (int xt = 0; xt < w; xt += RMX_WAVE * PX) {
        const int tw = min(w - xt, RMX_WAVE * PX);
        const int L = (tw + PX - 1) / PX;
        const int G = RMX_WAVE / L;
        const int lr = lane / L;
        const int g = lane - lr * L;
        const int gx = xt + g * PX;
        const int cnt = min(PX, w - gx);
        for (int r = r0 + lr; r < r1 && lr < G; r += G) {
            const uint8_t *p = simg + (size_t)(y1 + r) * row_stride + (size_t)(x1 + gx) * 3;
            uint32_t wd[6];
            load_realigned<7>(p, buf_end, wd);
            float v[3][PX];
            unpack8(wd, v);
#pragma unroll
            for (int k = 0; k < PX; k++) {
                if constexpr (KIND == COLOR_TWIST) {
                    twist_px(v[0][k], v[1][k], v[2][k], rcp, p0, p1, p2, p3);
                } else {
#pragma unroll
                    for (int c = 0; c < 3; c++) v[c][k] = __builtin_fmaf(v[c][k] - p2, p0, p1);
                }
            }
            store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, gx, cnt, v, false);
        }
    }
}

template <int KIND>
static KernelFn pick(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NCHW, KIND>;
            case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NCHW, KIND>;
            default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NCHW, KIND>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_color_kernel<float, RMX_NHWC, KIND>;
        case RMX_FP16: return (KernelFn)rmx_color_kernel<__half, RMX_NHWC, KIND>;
        default: return (KernelFn)rmx_color_kernel<uint8_t, RMX_NHWC, KIND>;
    }
}

KernelFn select_color_kernel(int kind, int dtype, int layout, const char **name) {
    *name = "rmx_color_kernel";
    return kind == COLOR_TWIST ? pick<COLOR_TWIST>(dtype, layout) : pick<COLOR_LINEAR>(dtype, layout);
}

}  // namespace rmx
