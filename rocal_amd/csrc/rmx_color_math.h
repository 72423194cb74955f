// Colour arithmetic shared by the colour kernel and by the resize kernels that run a colour node between the resize and the
// CropMirrorNormalize stage of a fused chain: the HSV twist of one pixel, its two LDS tables, and the chain stage itself.
#pragma once
#include "rmx_device.h"

namespace rmx {

// HSV -> RGB per hue sector: each output channel is one of V, q = V - V*S*f, p = V - V*S, t = p + V*S*f. All four have the form
// fma(sg, V*S*f, fma(nb, V*S, V)) with sg in {0,-1,+1} and nb in {0,-1}: a multiplication by 0 or +-1 is exact, so the two FMAs
// round exactly where the subtraction and the addition of the plain formulas round. The six coefficients of a sector come from
// a small LDS table indexed by the sector, which replaces the compare/select network (14 compares and selects per pixel).
//   sector:  0 1 2 3 4 5      r: V q p p t V      g: t V V q p p      b: p p t V V q
struct SectorRow {
    float sg[3], nb0;  // sg of r,g,b ; nb of r
    float nb1, nb2, pad0, pad1;  // nb of g,b
};
constexpr SectorRow sector_row(int hi) {
    // codes: 0 = V, 1 = q, 2 = p, 3 = t
    const int rc[6] = {0, 1, 2, 2, 3, 0}, gc[6] = {3, 0, 0, 1, 2, 2}, bc[6] = {2, 2, 3, 0, 0, 1};
    const int h = hi == 6 ? 0 : (hi > 5 ? 5 : hi);  // row 6 repeats row 0 (see the hue reduction), row 7 is never read
    const int code[3] = {rc[h], gc[h], bc[h]};
    float sg[3] = {0.0f, 0.0f, 0.0f}, nb[3] = {0.0f, 0.0f, 0.0f};
    for (int c = 0; c < 3; c++) {
        sg[c] = code[c] == 1 ? -1.0f : (code[c] == 3 ? 1.0f : 0.0f);
        nb[c] = code[c] >= 2 ? -1.0f : 0.0f;
    }
    return SectorRow{{sg[0], sg[1], sg[2]}, nb[0], nb[1], nb[2], 0.0f, 0.0f};
}

// How a hue comes back into [0, 6]. The hue of a pixel is num / delta + (0 | 2 | 4) + shift with |num / delta| <= 1 (to within
// a rounding), so for one sample, whose shift is one number, it lies in [shift - 1, shift + 5]: with shift below 1 it never
// reaches 6 and only "below 0: + 6" can happen, with shift above 1 it never falls below 0 and only "6 and above: - 6" can.
// Either is one comparison instead of two: hue >= t ? at : af is added, the same addition the two comparisons choose. A shift
// within 2e-5 of 1 keeps both comparisons (HUE_WRAP_BOTH): the host looks at the batch's shifts and picks the kernel
// (RMX_HUE_SHIFT_LOW / RMX_HUE_SHIFT_HIGH in rmx_common.h).
enum { HUE_WRAP_BOTH = 0, HUE_WRAP_ONE = 1 };
struct HueWrap {
    float t, at, af;
};
RMX_DEV HueWrap hue_wrap_of(float shift) {
    const bool low = shift < RMX_HUE_SHIFT_LOW;
    return HueWrap{low ? 0.0f : 6.0f, low ? 0.0f : -6.0f, low ? 6.0f : 0.0f};
}

// Branch-free: lanes of a wavefront hold pixels of different hue sectors, so
// branches would run every case one after the other under changing execution masks.
template <int WRAP = HUE_WRAP_BOTH>
RMX_DEV void twist_px(float &r, float &g, float &b, const float *rcp, const SectorRow *sect, float alpha, float beta, float shift, float shift2, float shift4, float satf,
                      float wrap_t = 0.0f, float wrap_at = 0.0f, float wrap_af = 0.0f) {
    // (the channel values as plain registers: knowing that they are converted bytes, the compiler subtracts the bytes as integers
    // for the hue numerator and converts the difference, one instruction more per pixel than subtracting the floats it has)
    asm("" : "+v"(r), "+v"(g), "+v"(b));
    const float cmax = __builtin_fmaxf(__builtin_fmaxf(r, g), b);
    const float cmin = __builtin_fminf(__builtin_fminf(r, g), b);
    const float delta = cmax - cmin;
    const float rd = rcp[(int)delta];      // 0 when delta == 0
    float s = delta * rcp[(int)cmax];
    // A grey pixel needs no case of its own: r == g == b makes it a "red is largest" pixel with g - b == 0.
    const bool is_r = cmax == r, is_g = cmax == g;
    const float d_gb = g - b, d_br = b - r, d_rg = r - g;  // (all three, then two selects: no branch)
    const float num = is_r ? d_gb : (is_g ? d_br : d_rg);
    // sextant offset 0 / 2 / 4 plus the hue shift, the three sums made once per sample
    const float add = is_r ? shift : (is_g ? shift2 : shift4);
    float hh = __builtin_fmaf(num, rd, add);
    // back into [0, 6]: one addition of +6, -6 or 0. A value just below zero can round to exactly 6.0 here; row 6 of the sector
    // table repeats row 0 and fract(6.0) is 0, which is the pixel a second reduction to 0.0 would give.
    if constexpr (WRAP == HUE_WRAP_ONE) hh = hh + (hh >= wrap_t ? wrap_at : wrap_af);
    else hh = hh + (hh < 0.0f ? 6.0f : (hh >= 6.0f ? -6.0f : 0.0f));
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

// The two tables of the twist: correctly rounded reciprocals of 0..255 (entry 0 is 0) and the sector coefficients. They are
// made by the compiler (IEEE division in a constant expression gives the same bits as the division on the device) and lie in
// device memory; a wavefront copies them into LDS, where the per-lane look-ups go.
struct __attribute__((aligned(16))) ColorTables {
    float rcp[256];
    SectorRow sect[8];
};
constexpr ColorTables make_color_tables() {
    ColorTables t{};
    for (int v = 0; v < 256; v++) t.rcp[v] = (v == 0) ? 0.0f : 1.0f / (float)v;
    for (int h = 0; h < 8; h++) t.sect[h] = sector_row(h);
    return t;
}
static __device__ const ColorTables rmx_color_tables_rom = make_color_tables();

// Copies the tables into LDS from one wavefront: 80 pieces of 16 bytes, one per lane and 16 more. Every wavefront of a
// workgroup writes the same values, so none has to wait for another: each reads only what it has written itself.
RMX_DEV void color_tables_fill(ColorTables *t, int lane) {
    static_assert(sizeof(ColorTables) == 80 * 16, "layout of the colour tables");
    const uint4 *src = reinterpret_cast<const uint4 *>(&rmx_color_tables_rom);
    uint4 *dst = reinterpret_cast<uint4 *>(t);
    dst[lane] = src[lane];
    if (lane < 16) dst[RMX_WAVE + lane] = src[RMX_WAVE + lane];
    wave_sync();
}

// Colour node in the middle of a fused chain resize(u8) -> colour(u8) -> CropMirrorNormalize: the values come in as the rounded
// u8 output of the resize node and leave as the rounded, saturated u8 output of the colour node.
//   CHAIN_LINEAR: fma(x - c2, c0, c1)   (Brightness: c0 = alpha, c1 = beta, c2 = 0; Contrast: c0 = factor, c1 = c2 = centre)
//   CHAIN_TWIST : twist_px with alpha = c0, beta = c1, hue shift in sextants = c2 (sh2, sh4 = c2 + 2, c2 + 4), saturation = c3
enum { CHAIN_NONE = 0, CHAIN_LINEAR = 1, CHAIN_TWIST = 2 };

template <int CHAIN>
RMX_DEV void chain_colour(float &o0, float &o1, float &o2, const float (&cp)[4], float sh2, float sh4, const ColorTables *t) {
    if constexpr (CHAIN == CHAIN_LINEAR) {
        o0 = __builtin_fmaf(o0 - cp[2], cp[0], cp[1]);
        o1 = __builtin_fmaf(o1 - cp[2], cp[0], cp[1]);
        o2 = __builtin_fmaf(o2 - cp[2], cp[0], cp[1]);
    } else if constexpr (CHAIN == CHAIN_TWIST) {
        twist_px(o0, o1, o2, t->rcp, t->sect, cp[0], cp[1], cp[2], sh2, sh4, cp[3]);
    }
    if constexpr (CHAIN != CHAIN_NONE) {
        o0 = round_u8(o0);
        o1 = round_u8(o1);
        o2 = round_u8(o2);
    }
}

}  // namespace rmx
