/*
 * rocal_oracle.c - CPU restatement of rocAL's augmentation hot path (TEST INFRASTRUCTURE ONLY;
 * see rocal_oracle.h for what pins each function). Plain C, scalar, OpenMP over samples.
 * Build with -ffp-contract=off: every fused multiply-add below is an explicit fmaf().
 */
#include "rocal_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------ fp16 */

/* IEEE binary32 -> binary16, round-to-nearest-even (HIP path of rocAL: __float2half,
 * rocAL/rocAL_hip/rocal_hip_kernels.cpp:210-212) or toward zero (CPU to_tensor,
 * rocAL/source/pipeline/master_graph.cpp:819-821). */
uint16_t orc_f32_to_f16(float v, int trunc) {
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
    }
    if (ax >= 0x477ff000u) { /* >= 65520: rounds to inf under RNE; trunc saturates to max finite */
        if (trunc) return (uint16_t)(sign | 0x7bffu);
        return (uint16_t)(sign | 0x7c00u);
    }
    if (trunc && ax >= 0x477fe000u) return (uint16_t)(sign | 0x7bffu);
    if (ax < 0x38800000u) { /* subnormal half or zero: value < 2^-14 */
        if (ax < 0x33000000u) { /* < 2^-25 */
            return (uint16_t)sign;
        }
        int e = (int)(ax >> 23);                     /* biased exponent, 102..112 */
        uint32_t m = (ax & 0x7fffffu) | 0x800000u;   /* 24-bit significand */
        int shift = 126 - e;                          /* result = m >> shift, in units of 2^-24 */
        uint32_t r = m >> shift;
        if (!trunc) {
            uint32_t rem = m & ((1u << shift) - 1u);
            uint32_t half = 1u << (shift - 1);
            if (rem > half || (rem == half && (r & 1u))) r++;
        }
        return (uint16_t)(sign | r);
    }
    uint32_t e = (ax >> 23) - 112u; /* half biased exponent */
    uint32_t m = ax & 0x7fffffu;
    uint32_t r = (e << 10) | (m >> 13);
    if (!trunc) {
        uint32_t rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    }
    return (uint16_t)(sign | r);
}

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    uint32_t x;
    if (e == 0) {
        if (m == 0) {
            x = sign;
        } else {
            int sh = 0;
            while (!(m & 0x400u)) { m <<= 1; sh++; }
            m &= 0x3ffu;
            x = sign | ((uint32_t)(113 - sh) << 23) | (m << 13);
        }
    } else if (e == 31) {
        x = sign | 0x7f800000u | (m << 13);
    } else {
        x = sign | ((e + 112u) << 23) | (m << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ------------------------------------------------------------------ stores */

static inline float round_u8(float v, unsigned flags) {
    /* default: round-to-nearest-even then saturate; in-tree HIP copies show both a
     * convert-and-pack (rocal_hip_kernels.cpp:425-430) and truncation (:499-502). */
    if (flags & ORC_F_ROUND_TRUNC) {
        v = fmaxf(fminf(v, 255.0f), 0.0f);
        return (float)(uint8_t)v;
    }
    v = rintf(v);
    v = v < 0.0f ? 0.0f : (v > 255.0f ? 255.0f : v);
    return v;
}

static inline size_t dst_index(const orc_dst *d, int n, int c, int y, int x) {
    if (d->layout == ORC_NCHW)
        return (((size_t)n * d->c + c) * d->hmax + y) * d->wmax + x;
    return (((size_t)n * d->hmax + y) * d->wmax + x) * d->c + c;
}

static inline void store(const orc_dst *d, size_t idx, float v, unsigned flags) {
    switch (d->dtype) {
        case ORC_FP32: ((float *)d->data)[idx] = v; break;
        case ORC_FP16: ((uint16_t *)d->data)[idx] = orc_f32_to_f16(v, (flags & ORC_F_FP16_TRUNC) != 0); break;
        default: ((uint8_t *)d->data)[idx] = (uint8_t)round_u8(v, flags); break;
    }
}

static inline const uint8_t *src_px(const orc_src *s, int n, int y, int x) {
    return s->data + (((size_t)n * s->hmax + y) * s->wmax + x) * s->c;
}

/* ------------------------------------------------------------------ CMN / crop / flip */

void orc_cmn_scale_bias(const float *mean, const float *stddev, int c, int n, float *scale, float *bias) {
    /* node_crop_mirror_normalize.cpp:56-61: offset = 1/std ; multiplier = -(mean*offset), fp32 */
    for (int i = 0; i < n; i++)
        for (int k = 0; k < c; k++) {
            float s = 1 / stddev[k];
            scale[i * c + k] = s;
            bias[i * c + k] = -(mean[k] * s);
        }
}

void orc_crop_mirror_normalize(const orc_src *src, const uint32_t *crop, const float *scale,
                               const float *bias, const uint32_t *mirror, const uint32_t *vflip,
                               const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x1 = (int)crop[n * 4 + 0], y1 = (int)crop[n * 4 + 1];
        int cw = (int)crop[n * 4 + 2], ch = (int)crop[n * 4 + 3];
        if (cw > dst->wmax) cw = dst->wmax;
        if (ch > dst->hmax) ch = dst->hmax;
        int m = mirror ? (mirror[n] != 0) : 0;
        int vf = vflip ? (vflip[n] != 0) : 0;
        for (int y = 0; y < ch; y++) {
            int sy = y1 + (vf ? ch - 1 - y : y);
            for (int x = 0; x < cw; x++) {
                int sx = x1 + (m ? cw - 1 - x : x);
                const uint8_t *p = src_px(src, n, sy, sx);
                for (int c = 0; c < C; c++) {
                    float v = (float)p[c];
                    if (scale) v = fmaf(v, scale[n * C + c], bias[n * C + c]);
                    store(dst, dst_index(dst, n, c, y, x), v, flags);
                }
            }
        }
    }
}

/* ------------------------------------------------------------------ resize */

/* rocal_hip_kernels.cpp:332-337 */
static inline float bilerp(float tl, float tr, float bl, float br, float wx, float wy) {
    float omx = 1.0f - wx, omy = 1.0f - wy;
    return fmaf(tl, omy * omx, fmaf(tr, omy * wx, fmaf(bl, wy * omx, br * wy * wx)));
}

static inline int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

typedef struct {
    int i0, i1;
    float w;
} lin_tap;

/* rocal_hip_kernels.cpp:311-330,340-343: src = dst*ratio + (ratio-1)/2 + roi.lo; floor; frac */
static void linear_taps(int lo, int len, int dlen, lin_tap *t, unsigned flags) {
    float ratio = (float)len / (float)dlen;
    float off = (ratio - 1.0f) * 0.5f;
    int hi = lo + len - 1;
    if (flags & ORC_F_BILINEAR_EDGE_QUIRK) hi -= 1;
    if (hi < lo) hi = lo;
    for (int d = 0; d < dlen; d++) {
        float s = (float)d * ratio;
        s = s + off;
        s = s + (float)lo;
        float f = floorf(s);
        t[d].w = s - f;
        t[d].i0 = clampi((int)f, lo, hi);
        t[d].i1 = clampi((int)f + 1, lo, hi);
    }
}

/* rocal_hip_kernels.cpp:487-512,555-558 */
typedef struct {
    int loc;     /* first tap (unclamped) */
    float w0;    /* loc - raw */
} tri_tap;

static void tri_setup(int lo, int len, int dlen, float *ratio, float *radius, float *fscale, int *ksize,
                      tri_tap *t) {
    *ratio = (float)len / (float)dlen;
    if (*ratio > 1.0f) {
        *radius = *ratio;
        *fscale = 1 / *ratio;
    } else {
        *radius = 1.0f;
        *fscale = 1.0f;
    }
    float off = (*ratio - 1) * 0.5f - *radius;
    *ksize = (int)ceilf(*radius * 2);
    for (int d = 0; d < dlen; d++) {
        float raw = (float)d * (*ratio);
        raw = raw + off;
        raw = raw + (float)lo;
        int loc = (int)ceilf(raw);
        t[d].loc = loc;
        t[d].w0 = (float)loc - raw;
    }
}

static inline float tri_coeff(float w0, float radius, int k, float fscale) {
    float c = 1 - fabsf((w0 - radius + (float)k) * fscale);
    return c < 0 ? 0 : c;
}

static void finish_px(const orc_dst *dst, int n, int c, int y, int x, float v, const float *scale,
                      const float *bias, int C, unsigned flags) {
    if (scale) {
        if (flags & ORC_F_QUANTIZE_U8) v = round_u8(v, flags);
        v = fmaf(v, scale[n * C + c], bias[n * C + c]);
    } else if (dst->dtype != ORC_UINT8 && (flags & ORC_F_QUANTIZE_U8)) {
        v = round_u8(v, flags);
    }
    store(dst, dst_index(dst, n, c, y, x), v, flags);
}

static void resize_one_linear(const orc_src *src, int n, const uint32_t *roi, int dw, int dh, int m,
                              const float *scale, const float *bias, const orc_dst *dst, unsigned flags) {
    const int C = src->c;
    lin_tap *tx = (lin_tap *)malloc(sizeof(lin_tap) * (size_t)(dw + dh));
    lin_tap *ty = tx + dw;
    linear_taps((int)roi[0], (int)roi[2], dw, tx, flags);
    linear_taps((int)roi[1], (int)roi[3], dh, ty, flags);
    for (int y = 0; y < dh; y++) {
        for (int x = 0; x < dw; x++) {
            const uint8_t *tl = src_px(src, n, ty[y].i0, tx[x].i0);
            const uint8_t *tr = src_px(src, n, ty[y].i0, tx[x].i1);
            const uint8_t *bl = src_px(src, n, ty[y].i1, tx[x].i0);
            const uint8_t *br = src_px(src, n, ty[y].i1, tx[x].i1);
            int ox = m ? dw - 1 - x : x;
            for (int c = 0; c < C; c++) {
                float v = bilerp((float)tl[c], (float)tr[c], (float)bl[c], (float)br[c], tx[x].w, ty[y].w);
                finish_px(dst, n, c, y, ox, v, scale, bias, C, flags);
            }
        }
    }
    free(tx);
}

static void resize_one_nearest(const orc_src *src, int n, const uint32_t *roi, int dw, int dh, int m,
                               const float *scale, const float *bias, const orc_dst *dst, unsigned flags) {
    /* DEFINED here: nearest = floor of the same half-pixel-centre source coordinate + 0.5 */
    const int C = src->c;
    lin_tap *tx = (lin_tap *)malloc(sizeof(lin_tap) * (size_t)(dw + dh));
    lin_tap *ty = tx + dw;
    linear_taps((int)roi[0], (int)roi[2], dw, tx, flags & ~ORC_F_BILINEAR_EDGE_QUIRK);
    linear_taps((int)roi[1], (int)roi[3], dh, ty, flags & ~ORC_F_BILINEAR_EDGE_QUIRK);
    for (int y = 0; y < dh; y++)
        for (int x = 0; x < dw; x++) {
            int sx = tx[x].w < 0.5f ? tx[x].i0 : tx[x].i1;
            int sy = ty[y].w < 0.5f ? ty[y].i0 : ty[y].i1;
            const uint8_t *p = src_px(src, n, sy, sx);
            int ox = m ? dw - 1 - x : x;
            for (int c = 0; c < C; c++) finish_px(dst, n, c, y, ox, (float)p[c], scale, bias, C, flags);
        }
    free(tx);
}

static void resize_one_triangular(const orc_src *src, int n, const uint32_t *roi, int dw, int dh, int m,
                                  const float *scale, const float *bias, const orc_dst *dst,
                                  unsigned flags) {
    const int C = src->c;
    int x0 = (int)roi[0], y0 = (int)roi[1], w = (int)roi[2], h = (int)roi[3];
    int xhi = x0 + w - 1, yhi = y0 + h - 1;
    float rx, ry, radx, rady, fsx, fsy;
    int kx, ky;
    tri_tap *tx = (tri_tap *)malloc(sizeof(tri_tap) * (size_t)(dw + dh));
    tri_tap *ty = tx + dw;
    tri_setup(x0, w, dw, &rx, &radx, &fsx, &kx, tx);
    tri_setup(y0, h, dh, &ry, &rady, &fsy, &ky, ty);

    if (flags & ORC_F_TRI_2D) {
        /* literal 2-D loop of rocal_hip_kernels.cpp:566-588 */
        for (int y = 0; y < dh; y++)
            for (int x = 0; x < dw; x++) {
                int ox = m ? dw - 1 - x : x;
                for (int c = 0; c < C; c++) {
                    float acc = 0.0f, rsum = 0.0f, csum = 0.0f;
                    for (int j = 0; j < ky; j++) {
                        int ri = clampi(ty[y].loc + j, y0, yhi);
                        float rc = tri_coeff(ty[y].w0, rady, j, fsy);
                        rsum += rc;
                        csum = 0;
                        for (int k = 0; k < kx; k++) {
                            int ci = clampi(tx[x].loc + k, x0, xhi);
                            float cc = tri_coeff(tx[x].w0, radx, k, fsx);
                            csum += cc;
                            float coeff = cc * rc;
                            acc += (float)src_px(src, n, ri, ci)[c] * coeff;
                        }
                    }
                    rsum = (rsum == 0.0f) ? 1.0f : rsum;
                    csum = (csum == 0.0f) ? 1.0f : csum;
                    acc *= 1 / (rsum * csum);
                    finish_px(dst, n, c, y, ox, acc, scale, bias, C, flags);
                }
            }
        free(tx);
        return;
    }

    /* separable evaluation (DEFINED here; algebraically the same weights):
     * horizontal pass over every source row a destination row touches, then vertical. */
    float *colsum = (float *)malloc(sizeof(float) * (size_t)dw);
    for (int x = 0; x < dw; x++) {
        float s = 0.0f;
        for (int k = 0; k < kx; k++) s += tri_coeff(tx[x].w0, radx, k, fsx);
        colsum[x] = (s == 0.0f) ? 1.0f : s;
    }
    float *hrow = (float *)malloc(sizeof(float) * (size_t)h * dw * C); /* rows y0..yhi */
    for (int r = 0; r < h; r++)
        for (int x = 0; x < dw; x++)
            for (int c = 0; c < C; c++) {
                float acc = 0.0f;
                for (int k = 0; k < kx; k++) {
                    int ci = clampi(tx[x].loc + k, x0, xhi);
                    acc = fmaf((float)src_px(src, n, y0 + r, ci)[c], tri_coeff(tx[x].w0, radx, k, fsx), acc);
                }
                hrow[((size_t)r * dw + x) * C + c] = acc;
            }
    for (int y = 0; y < dh; y++) {
        float rsum = 0.0f;
        for (int j = 0; j < ky; j++) rsum += tri_coeff(ty[y].w0, rady, j, fsy);
        rsum = (rsum == 0.0f) ? 1.0f : rsum;
        for (int x = 0; x < dw; x++) {
            int ox = m ? dw - 1 - x : x;
            float inv = 1 / (rsum * colsum[x]);
            for (int c = 0; c < C; c++) {
                float acc = 0.0f;
                for (int j = 0; j < ky; j++) {
                    int ri = clampi(ty[y].loc + j, y0, yhi) - y0;
                    acc = fmaf(hrow[((size_t)ri * dw + x) * C + c], tri_coeff(ty[y].w0, rady, j, fsy), acc);
                }
                acc *= inv;
                finish_px(dst, n, c, y, ox, acc, scale, bias, C, flags);
            }
        }
    }
    free(hrow);
    free(colsum);
    free(tx);
}

void orc_resize(const orc_src *src, const uint32_t *roi, const uint32_t *dst_w, const uint32_t *dst_h,
                int interp, const uint32_t *mirror, const float *scale, const float *bias,
                const orc_dst *dst, unsigned flags) {
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int dw = (int)dst_w[n], dh = (int)dst_h[n];
        if (dw > dst->wmax) dw = dst->wmax;
        if (dh > dst->hmax) dh = dst->hmax;
        if (dw <= 0 || dh <= 0 || roi[n * 4 + 2] == 0 || roi[n * 4 + 3] == 0) continue;
        int m = mirror ? (mirror[n] != 0) : 0;
        if (interp == ORC_INTERP_TRIANGULAR)
            resize_one_triangular(src, n, roi + n * 4, dw, dh, m, scale, bias, dst, flags);
        else if (interp == ORC_INTERP_NEAREST)
            resize_one_nearest(src, n, roi + n * 4, dw, dh, m, scale, bias, dst, flags);
        else
            resize_one_linear(src, n, roi + n * 4, dw, dh, m, scale, bias, dst, flags);
    }
}

/* ------------------------------------------------------------------ colour */

void orc_brightness(const orc_src *src, const uint32_t *roi, const float *alpha, const float *beta,
                    const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < C; c++)
                    store(dst, dst_index(dst, n, c, y, x), fmaf((float)p[c], alpha[n], beta[n]), flags);
            }
    }
}

void orc_contrast(const orc_src *src, const uint32_t *roi, const float *factor, const float *center,
                  const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < C; c++)
                    store(dst, dst_index(dst, n, c, y, x),
                          fmaf((float)p[c] - center[n], factor[n], center[n]), flags);
            }
    }
}

/* ---- streaming neighbours of the colour family. Their arithmetic lives only in RPP, which is absent from the
 * reference tree: each law below is DEFINED here from the parameter meanings the tree gives (PARITY UNPINNED). */

/* Gamma (vxExtRppGammaCorrection, node_gamma.cpp:42; gamma range 0.3..7, node_gamma.h:41): a 256-entry table per
 * sample, lut[i] = u8 store of powf(i/255, gamma)*255; every channel of every pixel goes through it. A float
 * destination receives the table value converted. */
void orc_gamma_lut(float gamma, uint8_t *lut, unsigned flags) {
    for (int i = 0; i < 256; i++) lut[i] = (uint8_t)round_u8(powf((float)i / 255.0f, gamma) * 255.0f, flags);
}

void orc_gamma(const orc_src *src, const uint32_t *roi, const float *gamma, const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        uint8_t lut[256];
        orc_gamma_lut(gamma[n], lut, flags);
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < C; c++) store(dst, dst_index(dst, n, c, y, x), (float)lut[p[c]], flags);
            }
    }
}

/* Exposure (vxExtRppExposure, node_exposure.cpp:42; factor range 0.15..0.95, node_exposure.h:42):
 * out = x * 2^factor, one fp32 product, u8 store. */
void orc_exposure(const orc_src *src, const uint32_t *roi, const float *factor, const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        const float m = exp2f(factor[n]);
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < C; c++) store(dst, dst_index(dst, n, c, y, x), (float)p[c] * m, flags);
            }
    }
}

/* ColorTemperature (vxExtRppColorTemperature, node_color_temperature.cpp:42; integer adjustment -99..99,
 * node_color_temperature.h:42-43): red + adj, green unchanged, blue - adj, saturating. */
void orc_color_temperature(const orc_src *src, const uint32_t *roi, const int32_t *adj, const orc_dst *dst, unsigned flags) {
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        const float d[3] = {(float)adj[n], 0.0f, -(float)adj[n]};
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < 3; c++) store(dst, dst_index(dst, n, c, y, x), (float)p[c] + d[c], flags);
            }
    }
}

/* Blend (vxExtRppBlend, node_blend.cpp:45; "output = input1*ratio + input2*(1-ratio)",
 * rocal_api_augmentation.h:371): evaluated as fmaf(a - b, ratio, b); a - b is exact for bytes, so the documented
 * value is rounded once. Both inputs share the first input's ROI (node_blend.cpp:45 passes only inputs[0]'s). */
void orc_blend(const orc_src *src1, const orc_src *src2, const uint32_t *roi, const float *ratio, const orc_dst *dst, unsigned flags) {
    const int C = src1->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src1->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src1, n, y0 + y, x0 + x);
                const uint8_t *q = src_px(src2, n, y0 + y, x0 + x);
                for (int c = 0; c < C; c++)
                    store(dst, dst_index(dst, n, c, y, x), fmaf((float)p[c] - (float)q[c], ratio[n], (float)q[c]), flags);
            }
    }
}

/* Normalize (vxExtRppNormalize, effects_augmentations/node_normalize.cpp:31-113) for image tensors; law DEFINED here (the arithmetic
 * lives in RPP): statistics over height and width (axis_mask 3: per channel) or height, width and channels (7: per sample), from
 * exact integer moments: mean = sum / count, stddev = sqrt(sum (x - mean)^2 / count) in double, then fp32
 * a = scale / stddev (0 when stddev is 0), b = fmaf(-mean, a, shift), out = fmaf(x, a, b). */
void orc_normalize(const orc_src *src, const uint32_t *roi, unsigned axis_mask, const float *mean, const float *stddev, unsigned n_stats,
                   float scale, float shift, const orc_dst *dst, unsigned flags) {
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        unsigned long long sum[3] = {0, 0, 0}, sq[3] = {0, 0, 0};
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < 3; c++) {
                    sum[c] += p[c];
                    sq[c] += (unsigned)p[c] * p[c];
                }
            }
        float a[3], b[3];
        for (int c = 0; c < 3; c++) {
            double cnt = (double)w * (double)h, s1 = (double)sum[c], s2 = (double)sq[c];
            if (axis_mask == 7u) {
                cnt *= 3.0;
                s1 = (double)(sum[0] + sum[1] + sum[2]);
                s2 = (double)(sq[0] + sq[1] + sq[2]);
            }
            float m = mean ? mean[n_stats == 3 ? c : 0] : 0.0f, sd = stddev ? stddev[n_stats == 3 ? c : 0] : 1.0f;
            if (cnt > 0.0) {
                const double md = mean ? (double)m : s1 / cnt;
                if (!mean) m = (float)md;
                if (!stddev) {
                    double var = (s2 - 2.0 * md * s1 + cnt * md * md) / cnt;
                    if (var < 0.0) var = 0.0;
                    sd = (float)sqrt(var);
                }
            }
            a[c] = sd != 0.0f ? scale / sd : 0.0f;
            b[c] = fmaf(-m, a[c], shift);
        }
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                for (int c = 0; c < 3; c++) store(dst, dst_index(dst, n, c, y, x), fmaf((float)p[c], a[c], b[c]), flags);
            }
    }
}

/* hue in degrees -> shift in sextants, reduced to [0,6] */
static float hue_shift_sextants(float hue_deg, unsigned flags) {
    if (flags & ORC_F_HUE_INT_TRUNC) hue_deg = (float)((int)hue_deg % 360);
    float s = fmodf(hue_deg, 360.0f);
    if (s < 0.0f) s += 360.0f;
    return s / 60.0f;
}

void orc_color_twist(const orc_src *src, const uint32_t *roi, const float *alpha, const float *beta,
                     const float *hue, const float *sat, const orc_dst *dst, unsigned flags) {
    /* DEFINED here (RPP's HSV formulation restated on the 0..255 scale; beta is additive on
     * that scale, rocAL/include/augmentations/color_augmentations/node_color_twist.h:44-47). */
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        float shift = hue_shift_sextants(hue[n], flags);
        float a = alpha[n], b = beta[n], sf = sat[n];
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++) {
                const uint8_t *p = src_px(src, n, y0 + y, x0 + x);
                float rf = (float)p[0], gf = (float)p[1], bf = (float)p[2];
                float cmax = fmaxf(fmaxf(rf, gf), bf);
                float cmin = fminf(fminf(rf, gf), bf);
                float delta = cmax - cmin;
                float num = 0.0f, add = 0.0f, rd = 0.0f, s = 0.0f;
                if (delta != 0.0f) {
                    rd = 1.0f / delta;
                    s = delta * (1.0f / cmax);
                    if (cmax == rf) {
                        num = gf - bf;
                        add = 0.0f;
                    } else if (cmax == gf) {
                        num = bf - rf;
                        add = 2.0f;
                    } else {
                        num = rf - gf;
                        add = 4.0f;
                    }
                }
                float hh = fmaf(num, rd, add + shift);
                if (hh < 0.0f) hh += 6.0f;
                if (hh >= 6.0f) hh -= 6.0f;
                s = s * sf;
                s = fminf(fmaxf(s, 0.0f), 1.0f);
                int hi = (int)hh;
                float hf = hh - (float)hi;
                float vsat = cmax * s;
                float vsatf = vsat * hf;
                float pp = cmax - vsat;
                float qq = cmax - vsatf;
                float tt = pp + vsatf;
                float r, g, bl;
                switch (hi) {
                    case 0: r = cmax; g = tt; bl = pp; break;
                    case 1: r = qq; g = cmax; bl = pp; break;
                    case 2: r = pp; g = cmax; bl = tt; break;
                    case 3: r = pp; g = qq; bl = cmax; break;
                    case 4: r = tt; g = pp; bl = cmax; break;
                    default: r = cmax; g = pp; bl = qq; break;
                }
                store(dst, dst_index(dst, n, 0, y, x), fmaf(r, a, b), flags);
                store(dst, dst_index(dst, n, 1, y, x), fmaf(g, a, b), flags);
                store(dst, dst_index(dst, n, 2, y, x), fmaf(bl, a, b), flags);
            }
    }
}

/* ------------------------------------------------------------------ warp / rotate */

void orc_affine_from_rocal(const float a[6], float m[6]) {
    /* rocAL fills x0,y0,x1,y1,o0,o1 (node_warp_affine.cpp:43-48); DEFINED here as
     * M = [[x0, x1, o0], [y0, y1, o1]] */
    m[0] = a[0]; m[1] = a[2]; m[2] = a[4];
    m[3] = a[1]; m[4] = a[3]; m[5] = a[5];
}

void orc_rotate_matrix(float angle_deg, float m[6]) {
    /* forward map of meta_node_rotate.cpp:53-77 is [[c, s], [-s, c]] about the centres,
     * so destination->source uses its transpose. */
    float rad = angle_deg * 0.017453292519943295f;
    float c = cosf(rad), s = sinf(rad);
    m[0] = c; m[1] = -s; m[2] = 0.0f;
    m[3] = s; m[4] = c;  m[5] = 0.0f;
}

void orc_warp_affine(const orc_src *src, const uint32_t *roi, const float *affine, int interp,
                     const uint32_t *dst_w, const uint32_t *dst_h, const orc_dst *dst, unsigned flags) {
    const int C = src->c;
#pragma omp parallel for schedule(dynamic)
    for (int n = 0; n < src->n; n++) {
        int x0 = (int)roi[n * 4], y0 = (int)roi[n * 4 + 1], w = (int)roi[n * 4 + 2], h = (int)roi[n * 4 + 3];
        int dw = (int)dst_w[n], dh = (int)dst_h[n];
        if (dw > dst->wmax) dw = dst->wmax;
        if (dh > dst->hmax) dh = dst->hmax;
        if (w <= 0 || h <= 0) continue;
        const float *m = affine + n * 6;
        int xhi = x0 + w - 1, yhi = y0 + h - 1;
        float dcx = (float)(dw >> 1), dcy = (float)(dh >> 1);
        float scx = (float)(x0 + (w >> 1)), scy = (float)(y0 + (h >> 1));
        for (int y = 0; y < dh; y++)
            for (int x = 0; x < dw; x++) {
                float xr = (float)x - dcx, yr = (float)y - dcy;
                float sx = fmaf(xr, m[0], fmaf(yr, m[1], m[2])) + scx;
                float sy = fmaf(xr, m[3], fmaf(yr, m[4], m[5])) + scy;
                float out[4] = {0, 0, 0, 0};
                if (interp == ORC_INTERP_NEAREST) {
                    float fx = floorf(sx + 0.5f), fy = floorf(sy + 0.5f);
                    if (!(fx < (float)x0 || fy < (float)y0 || fx > (float)xhi || fy > (float)yhi)) {
                        const uint8_t *p = src_px(src, n, (int)fy, (int)fx);
                        for (int c = 0; c < C; c++) out[c] = (float)p[c];
                    }
                } else {
                    float fx = floorf(sx), fy = floorf(sy);
                    /* out-of-ROI rule shaped after rocal_hip_kernels.cpp:396-397 */
                    if (!(fx < (float)x0 || fy < (float)y0 || fx > (float)xhi || fy > (float)yhi)) {
                        float wx = sx - fx, wy = sy - fy;
                        int ix0 = (int)fx, iy0 = (int)fy;
                        int ix1 = ix0 + 1 > xhi ? xhi : ix0 + 1;
                        int iy1 = iy0 + 1 > yhi ? yhi : iy0 + 1;
                        const uint8_t *tl = src_px(src, n, iy0, ix0), *tr = src_px(src, n, iy0, ix1);
                        const uint8_t *bl = src_px(src, n, iy1, ix0), *br = src_px(src, n, iy1, ix1);
                        for (int c = 0; c < C; c++)
                            out[c] = bilerp((float)tl[c], (float)tr[c], (float)bl[c], (float)br[c], wx, wy);
                    }
                }
                for (int c = 0; c < C; c++) store(dst, dst_index(dst, n, c, y, x), out[c], flags);
            }
    }
}

/* ------------------------------------------------------------------ to_tensor */

void orc_to_tensor(const uint8_t *src, int n, int h, int w, int c, const float mul[3], const float add[3],
                   int reverse_channels, const orc_dst *dst, unsigned flags) {
    /* master_graph.cpp:751-753 (_mm256_fmadd_ps) / rocal_hip_kernels.cpp:161-165 */
#pragma omp parallel for schedule(dynamic)
    for (int i = 0; i < n; i++)
        for (int y = 0; y < dst->hmax; y++)
            for (int x = 0; x < dst->wmax; x++)
                for (int k = 0; k < c; k++) {
                    int sk = reverse_channels ? c - 1 - k : k;
                    float v = (float)src[(((size_t)i * h + y) * w + x) * c + sk];
                    store(dst, dst_index(dst, i, k, y, x), fmaf(v, mul[k], add[k]), flags);
                }
}

/* ------------------------------------------------------------------ parameter laws */

void orc_mt19937_seed(orc_mt19937 *g, uint32_t seed) {
    g->mt[0] = seed;
    for (int i = 1; i < 624; i++) g->mt[i] = 1812433253u * (g->mt[i - 1] ^ (g->mt[i - 1] >> 30)) + (uint32_t)i;
    g->idx = 624;
}

uint32_t orc_mt19937_next(orc_mt19937 *g) {
    if (g->idx >= 624) {
        for (int i = 0; i < 624; i++) {
            uint32_t y = (g->mt[i] & 0x80000000u) | (g->mt[(i + 1) % 624] & 0x7fffffffu);
            g->mt[i] = g->mt[(i + 397) % 624] ^ (y >> 1) ^ ((y & 1u) ? 0x9908b0dfu : 0u);
        }
        g->idx = 0;
    }
    uint32_t y = g->mt[g->idx++];
    y ^= y >> 11;
    y ^= (y << 7) & 0x9d2c5680u;
    y ^= (y << 15) & 0xefc60000u;
    y ^= y >> 18;
    return y;
}

/* C++ [rand.util.seedseq] generate(), for 32-bit outputs */
void orc_seed_seq_generate(const uint32_t *v, int s, uint32_t *out, int n) {
    if (n <= 0) return;
    for (int i = 0; i < n; i++) out[i] = 0x8b8b8b8bu;
    int t = (n >= 623) ? 11 : (n >= 68) ? 7 : (n >= 39) ? 5 : (n >= 7) ? 3 : (n - 1) / 2;
    int p = (n - t) / 2, q = p + t;
    int m = (s + 1 > n) ? s + 1 : n;
#define T_(x) ((x) ^ ((x) >> 27))
    for (int k = 0; k < m; k++) {
        uint32_t a = out[k % n] ^ out[(k + p) % n] ^ out[(k + n - 1) % n];
        uint32_t r1 = 1664525u * T_(a);
        uint32_t r2 = r1;
        if (k == 0) r2 += (uint32_t)s;
        else if (k <= s) r2 += (uint32_t)(k % n) + v[k - 1];
        else r2 += (uint32_t)(k % n);
        out[(k + p) % n] += r1;
        out[(k + q) % n] += r2;
        out[k % n] = r2;
    }
    for (int k = m; k < m + n; k++) {
        uint32_t a = out[k % n] + out[(k + p) % n] + out[(k + n - 1) % n];
        uint32_t r3 = 1566083941u * T_(a);
        uint32_t r4 = r3 - (uint32_t)(k % n);
        out[(k + p) % n] ^= r3;
        out[(k + q) % n] ^= r4;
        out[k % n] = r4;
    }
#undef T_
}

float orc_uniform_rand_f32(orc_mt19937 *g, float start, float end) {
    uint32_t val = orc_mt19937_next(g); /* drawn even when start == end (parameter_random.h:61) */
    if (end < start) end = start;
    if (start == end) return start;
    return (float)(((double)val / (double)4294967295u) * ((double)end - (double)start) + (double)start);
}

int orc_uniform_rand_i32(orc_mt19937 *g, int start, int end) {
    uint32_t val = orc_mt19937_next(g);
    if (end < start) end = start;
    if (start == end) return start;
    return (int)(((double)val / (double)4294967295u) * ((double)end - (double)start) + (double)start);
}

int orc_custom_rand_index(orc_mt19937 *g, const double *freq, int size) {
    if (size == 1) return 0; /* no draw when single valued (parameter_random.h:178-181) */
    double sum = 0;
    for (int i = 0; i < size; i++)
        if (freq[i] >= 0) sum += freq[i];
    double r = (double)orc_mt19937_next(g) / (double)4294967295u;
    double acc = 0;
    for (int i = 0; i < size; i++) {
        /* note: the reference's copy_if compacts non-negative entries; callers here pass
         * non-negative frequencies only */
        acc += freq[i] / sum;
        if (acc > r) return i; /* upper_bound: first cdf entry strictly greater */
    }
    return size; /* r == 1.0 exactly: one past the end, as upper_bound returns */
}

void orc_fixed_crop(uint32_t roi_w, uint32_t roi_h, uint32_t crop_w, uint32_t crop_h, int is_fixed_anchor,
                    float anchor_x, float anchor_y, uint32_t x1, uint32_t y1, uint32_t out[4]) {
    uint32_t cw = (crop_w <= roi_w && crop_w > 0) ? crop_w : roi_w;
    uint32_t ch = (crop_h <= roi_h && crop_h > 0) ? crop_h : roi_h;
    uint32_t ox, oy;
    if (is_fixed_anchor) {
        ox = (uint32_t)(size_t)nearbyintf(anchor_x * (float)(roi_w - cw));
        oy = (uint32_t)(size_t)nearbyintf(anchor_y * (float)(roi_h - ch));
    } else {
        ox = (x1 >= roi_w) ? 0 : x1;
        oy = (y1 >= roi_h) ? 0 : y1;
    }
    uint32_t x2 = ox + cw, y2 = oy + ch;
    if (x2 > roi_w) x2 = roi_w;
    if (y2 > roi_h) y2 = roi_h;
    out[0] = ox; out[1] = oy; out[2] = cw; out[3] = ch;
    (void)x2; (void)y2; /* the reference clamps x2/y2 but publishes x1,y1,cw,ch */
}

void orc_fparam_uniform(orc_fparam *p, float lo, float hi, uint32_t seed) {
    orc_mt19937_seed(&p->g, seed);
    p->lo = lo;
    p->hi = hi < lo ? lo : hi;
    p->simple = 0;
    p->value = orc_uniform_rand_f32(&p->g, p->lo, p->hi);
}

void orc_fparam_simple(orc_fparam *p, float value) {
    p->simple = 1;
    p->value = value;
}

float orc_fparam_renew(orc_fparam *p) {
    if (!p->simple) p->value = orc_uniform_rand_f32(&p->g, p->lo, p->hi);
    return p->value;
}

void orc_random_crop(orc_fparam *area, orc_fparam *aspect, orc_fparam *x_drift, orc_fparam *y_drift, uint32_t W,
                     uint32_t H, uint32_t out[4]) {
    const float ar_lo = 0.75f, ar_hi = 1.333f; /* parameter_random_crop.h:43 */
    uint32_t cw = 0, ch = 0, x = 0, y = 0;
    int ok = 0;
    for (int attempt = 0; attempt < 5 && !ok; attempt++) { /* :50 */
        float a = orc_fparam_renew(area);
        float r = orc_fparam_renew(aspect);
        float t32 = a * (float)H; /* float arithmetic, left to right, widened to double on assignment (:64) */
        t32 = t32 * (float)W;
        double target = (double)t32;
        cw = (uint32_t)(size_t)sqrt(target * (double)r);
        ch = (uint32_t)(size_t)sqrt(target * (double)(1 / r));
        if (ch < H && cw < W) { /* strictly smaller (:55-57) */
            float xd = orc_fparam_renew(x_drift);
            orc_fparam_renew(y_drift);
            float yd = orc_fparam_renew(y_drift); /* renewed twice (:70-72) */
            x = (uint32_t)(size_t)(xd * (float)(W - cw));
            y = (uint32_t)(size_t)(yd * (float)(H - ch));
            ok = 1;
        }
    }
    if (!ok) { /* central crop, aspect ratio pulled into range (:81-94) */
        float in_ratio = (float)W / (float)H;
        if (in_ratio < ar_lo) {
            cw = W;
            ch = (uint32_t)((float)cw / ar_lo);
        } else if (in_ratio > ar_hi) {
            ch = H;
            cw = (uint32_t)((float)ch * ar_hi);
        } else {
            ch = H;
            cw = W;
        }
        x = (W - cw) / 2;
        y = (H - ch) / 2;
    }
    out[0] = x; out[1] = y; out[2] = cw; out[3] = ch;
}

void orc_factor_crop(orc_fparam *h_factor, orc_fparam *w_factor, orc_fparam *x_drift, orc_fparam *y_drift, uint32_t W,
                     uint32_t H, uint32_t out[4]) {
    float fh = orc_fparam_renew(h_factor);
    float fw = orc_fparam_renew(w_factor);
    uint32_t cw = (uint32_t)(size_t)(fw * (float)W);
    uint32_t ch = (uint32_t)(size_t)(fh * (float)H);
    float xd = orc_fparam_renew(x_drift);
    float yd = orc_fparam_renew(y_drift);
    out[0] = (uint32_t)(size_t)(xd * (float)(W - cw));
    out[1] = (uint32_t)(size_t)(yd * (float)(H - ch));
    out[2] = cw;
    out[3] = ch;
}

void orc_resize_out_size(unsigned sw, unsigned sh, unsigned dw, unsigned dh, int mode, unsigned max_w,
                         unsigned max_h, unsigned *out_w, unsigned *out_h) {
    int has_max = (max_w | max_h) > 0;
    if (mode == 1) { /* stretch */
        if (!dw) dw = sw;
        if (!dh) dh = sh;
        if (has_max) {
            if (max_w && dw > max_w) dw = max_w;
            if (max_h && dh > max_h) dh = max_h;
        }
    } else if (mode == 0) { /* default */
        if (!dw && dh) dw = (unsigned)lroundf((float)sw * ((float)dh / (float)sh));
        else if (!dh && dw) dh = (unsigned)lroundf((float)sh * ((float)dw / (float)sw));
        if (has_max) {
            if (max_w && dw > max_w) dw = max_w;
            if (max_h && dh > max_h) dh = max_h;
        }
    } else {
        float scale = 1.0f;
        float scale_w = (float)dw / (float)sw, scale_h = (float)dh / (float)sh;
        if (mode == 2) scale = scale_w > scale_h ? scale_w : scale_h;
        else if (mode == 3)
            scale = (scale_w > 0 && scale_h > 0) ? (scale_w < scale_h ? scale_w : scale_h)
                                                 : ((scale_w > 0) ? scale_w : scale_h);
        if (has_max) {
            if (max_w) { float s = (float)max_w / (float)sw; if (s < scale) scale = s; }
            if (max_h) { float s = (float)max_h / (float)sh; if (s < scale) scale = s; }
        }
        if (scale_h != scale || !dh) dh = (unsigned)lroundf((float)sh * scale);
        if (scale_w != scale || !dw) dw = (unsigned)lroundf((float)sw * scale);
    }
    *out_w = dw;
    *out_h = dh;
}
