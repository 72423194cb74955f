// K2: ROI crop -> bilinear (or nearest) resize -> [u8 quantise] -> [mirror] -> [normalise]
//     -> layout transpose -> cast, in one pass. Serves Resize / CropResize / ROIResize /
//     ResizeCropMirror / ResizeMirrorNormalize and the fused RandomResizedCrop + CMN chain.
//
// Scheduling is wavefront-granular: every wavefront owns a strip of output rows of one sample
// and a private slice of LDS; there is no workgroup barrier anywhere. The wave walks down its
// strip in steps of G output rows (G = 64 / lanes-per-row) and keeps a ring of staged source
// rows in LDS, so every source row is fetched once per strip:
//   stage    rows entering the window are read with dword-aligned 128-bit global loads
//            (12 useful bytes = 4 packed pixels per lane; the row base is wave-uniform, so the
//            per-lane address is one precomputed offset) and expanded to one dword per pixel,
//            which makes the gather bank-friendly and free of byte addressing;
//   gather   two adjacent-dword LDS reads per neighbour row and pixel, fp32 blend in the
//            reference's FMA order, epilogue, eight pixels per lane written with 128-bit stores.
// The loads of step k+1 are issued before the arithmetic of step k and committed to LDS after
// it, so HBM latency overlaps the blend. HBM-bound by design: window bytes in, tensor bytes out.
#pragma once
#include "rmx_device.h"
#include "rmx_color_math.h"
#include "rmx_launch.h"

namespace rmx {

extern __shared__ uint32_t rmx_lds[];

constexpr int NL = 8;   // 128-bit loads a lane may hold in flight across the blend of a step

// source coordinate of resized index u (rocal bilinear law: u*ratio + (ratio-1)/2 + roi.lo)
RMX_DEV float src_coord(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}

// Everything the staging of one x-tile needs; all members are wave-uniform.
struct StageCtx {
    const uint8_t *base4;  // sample base rounded down to 4 bytes (global memory)
    uint32_t skew;         // sample base - base4
    uint32_t lim;          // bytes from base4 to the end of the batch buffer (saturated to 32 bits)
    uint32_t row_stride;   // bytes
    int cs;                // first staged source column
    int items;             // 4-pixel items per row
    int ipl;               // items per lane per row = ceil(items/64)
    int pitch;             // LDS row pitch in dwords
    int ylo, yhi;          // ROI rows
    int R;                 // ring rows
};

// byte offset (from base4) of the first staged pixel of virtual source row v
RMX_DEV uint32_t stage_row_offset(const StageCtx &S, int v) {
    const int ysrc = max(min(v, S.yhi), S.ylo);
    return (uint32_t)ysrc * S.row_stride + (uint32_t)S.cs * 3u + S.skew;
}

// Issue the loads of staging items [first, first+NL) of the row set starting at virtual row
// new_lo; item t is (row t / ipl, chunk t % ipl); a lane handles 4-pixel item j = lane + 64*chunk
// of its row with one dword-aligned 128-bit load (uniform base + 32-bit lane offset).
RMX_DEV void stage_issue(const StageCtx &S, int lane, int new_lo, int nit, int first, uint32_t (&raw)[NL][4]) {
    int q = first / S.ipl, c = first - q * S.ipl;
#pragma unroll
    for (int t = 0; t < NL; t++) {
        if (first + t < nit) {
            const uint32_t ro4 = stage_row_offset(S, new_lo + q) & ~3u;
            const int j = lane + RMX_WAVE * c;
            if (j < S.items) {
                const uint32_t vo = ro4 + 12u * (uint32_t)j;
                if (ro4 + 12u * (uint32_t)S.items + 8u <= S.lim) {  // row segment + realign slack inside the batch
                    u32x4_a4 v = *reinterpret_cast<const u32x4_a4 *>(S.base4 + vo);
                    raw[t][0] = v.x; raw[t][1] = v.y; raw[t][2] = v.z; raw[t][3] = v.w;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) raw[t][i] = (vo + 4u * i < S.lim) ? *reinterpret_cast<const uint32_t *>(S.base4 + vo + 4u * i) : 0u;
                }
            }
            if (++c == S.ipl) {
                c = 0;
                q++;
            }
        }
    }
}

// Expand the loaded items and write them to their ring slots.
RMX_DEV void stage_commit(const StageCtx &S, uint32_t *lds, int lane, int new_lo, int slot_new, int nit, int first,
                          const uint32_t (&raw)[NL][4]) {
    int q = first / S.ipl, c = first - q * S.ipl;
#pragma unroll
    for (int t = 0; t < NL; t++) {
        if (first + t < nit) {
            const uint32_t phase = stage_row_offset(S, new_lo + q) & 3u;
            int sl = slot_new + q;
            if (sl >= S.R) sl -= S.R;
            const int j = lane + RMX_WAVE * c;
            if (j < S.items) *reinterpret_cast<uint4 *>(lds + sl * S.pitch + 4 + 4 * j) = expand4(raw[t], phase);
            if (++c == S.ipl) {
                c = 0;
                q++;
            }
        }
    }
}

// CHAIN: a colour node between the (quantised) resize and the normalisation, see chain_colour().
template <typename T, int LAYOUT, bool NORM, bool QUANT, bool NEAREST, int CHAIN = CHAIN_NONE>
__global__ void __launch_bounds__(256) rmx_resize_kernel(RmxKArgs a) {
    static_assert(CHAIN == CHAIN_NONE || (QUANT && !NEAREST), "a colour node in the chain reads the u8 output of a bilinear resize node");
    __shared__ __attribute__((aligned(16))) float chain_tables[CHAIN == CHAIN_TWIST ? sizeof(ColorTables) / 4 : 4];
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, gridDim.x) * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, strip;
    wave_to_sample(a, wave, s, strip);
    const RmxSample &P = a.table[s];

    const int dw = P.dst_w, dh = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= dh || dw <= 0) return;
    const int r1 = min(r0 + srows, dh);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;

    const int xlo = P.src_x, ylo = P.src_y;
    // last column / row a tap may read: the window's last one, or the one before it under the reference's device edge rule
    const int edge = (int)((P.flags / RMX_S_EDGE_REF) & 1u);
    const int xhi = max(xlo + P.src_w - 1 - edge, xlo), yhi = max(ylo + P.src_h - 1 - edge, ylo);
    const float rx = P.rx, ry = P.ry;
    const float offx = (rx - 1.0f) * 0.5f, offy = (ry - 1.0f) * 0.5f;
    const float fxlo = (float)xlo, fylo = (float)ylo;
    const int pcx = P.pc_x, pcy = P.pc_y;

    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *lds = rmx_lds + (size_t)wib * (a.lds_bytes >> 2);

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }
    // colour node of a fused chain: its four parameters travel in the (otherwise unused) affine fields of the row
    const float cp[4] = {P.m[0], P.m[1], P.m[2], P.m[3]};
    const float sh2 = cp[2] + 2.0f, sh4 = cp[2] + 4.0f;
    const ColorTables *ctab = reinterpret_cast<const ColorTables *>(chain_tables);
    if constexpr (CHAIN == CHAIN_TWIST) color_tables_fill(reinterpret_cast<ColorTables *>(chain_tables), lane);

    StageCtx S;
    {
        const uint8_t *simg = sample_base(a, s, S.row_stride);
        S.skew = (uint32_t)((uintptr_t)simg & 3u);
        S.base4 = simg - S.skew;
        const uint64_t left = (uint64_t)((a.src + a.src_bytes) - S.base4);
        S.lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;
    }
    S.ylo = ylo;
    S.yhi = yhi;
    S.R = P.strip_rows;
    const int R = S.R;

    const int tile_w = a.aux1;  // output columns per x-tile (multiple of PX, <= 64*PX)
    for (int xt = 0; xt < dw; xt += tile_w) {
        const int tw = min(dw - xt, tile_w);
        const int L = (tw + PX - 1) / PX;
        const int G = RMX_WAVE / L;
        const int lr = lane / L;
        const int g = lane - lr * L;
        const int t0 = xt + g * PX;  // first window-relative column of the group
        const int cnt = min(PX, dw - t0);
        const bool lane_on = lr < G && cnt > 0;

        // tile-wide source column range (wave-uniform)
        const int u_first = pcx + xt, u_last = pcx + xt + tw - 1;
        const int ixmin = (int)floorf(src_coord(u_first, rx, offx, fxlo));
        const int ixmax = (int)floorf(src_coord(u_last, rx, offx, fxlo));
        const int cs = max(min(ixmin, xhi), xlo);
        const int ce = max(min(ixmax + 1, xhi), xlo);
        const int nc = ce - cs + 1;
        const bool rep_l = ixmin < xlo, rep_r = ixmax + 1 > xhi;
        S.cs = cs;
        S.items = (nc + 3) >> 2;
        S.ipl = (S.items + RMX_WAVE - 1) / RMX_WAVE;
        S.pitch = 4 + S.items * 4 + 4;
        const int pitch = S.pitch;

        // per-lane column taps, fixed for the whole strip (LDS dword index of the left neighbour)
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

        // ---- first step: stage its whole window
        int a_k = (int)floorf(src_coord(pcy + r0, ry, offy, fylo));
        int b_k = (int)floorf(src_coord(pcy + min(r0 + G, r1) - 1, ry, offy, fylo)) + 1;
        int base_slot = 0;
        uint32_t raw[NL][4];
        {
            const int nnew = b_k - a_k + 1, nit = nnew * S.ipl;
            for (int first = 0; first < nit; first += NL) {
                stage_issue(S, lane, a_k, nit, first, raw);
                stage_commit(S, lds, lane, a_k, 0, nit, first, raw);
            }
            wave_sync();
            if ((rep_l || rep_r) && lane < nnew) {
                uint32_t *row = lds + lane * pitch;
                if (rep_l) row[3] = row[4];
                if (rep_r) row[4 + nc] = row[4 + nc + 1] = row[4 + nc - 1];  // two: under the device edge rule a left tap can lie one beyond
            }
            wave_sync();
        }

        for (int rs = r0; rs < r1; rs += G) {
            const int re = min(rs + G, r1) - 1;
            // ---- next step's window; issue its loads before this step's arithmetic
            const bool has_next = rs + G < r1;
            int a_n = a_k, b_n = b_k, new_lo = 0, nnew = 0, nit = 0, base_slot_n = base_slot, slot_new = 0;
            if (has_next) {
                a_n = (int)floorf(src_coord(pcy + rs + G, ry, offy, fylo));
                b_n = (int)floorf(src_coord(pcy + min(rs + 2 * G, r1) - 1, ry, offy, fylo)) + 1;
                base_slot_n = base_slot + (a_n - a_k);
                while (base_slot_n >= R) base_slot_n -= R;
                new_lo = max(b_k + 1, a_n);
                nnew = b_n - new_lo + 1;
                nit = nnew * S.ipl;
                slot_new = base_slot_n + (new_lo - a_n);
                if (slot_new >= R) slot_new -= R;
                stage_issue(S, lane, new_lo, nit, 0, raw);
            }

            // ---- gather + blend + epilogue for rows rs..re
            const int r = rs + lr;
            if (lane_on && r <= re) {
                float sy = src_coord(pcy + r, ry, offy, fylo);
                float fy = floorf(sy);
                float wy = sy - fy;
                int s0 = base_slot + ((int)fy - a_k);
                if (s0 >= R) s0 -= R;
                int s1 = s0 + 1;
                if (s1 >= R) s1 -= R;
                const uint32_t *row0 = lds + s0 * pitch;
                const uint32_t *row1 = lds + s1 * pitch;
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
                if constexpr (CHAIN != CHAIN_NONE) {
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        float o0 = __builtin_rintf(v[0][k]), o1 = __builtin_rintf(v[1][k]), o2 = __builtin_rintf(v[2][k]);
                        chain_colour<CHAIN>(o0, o1, o2, cp, sh2, sh4, ctab);
                        v[0][k] = __builtin_fmaf(o0, sc[0], bi[0]);
                        v[1][k] = __builtin_fmaf(o1, sc[1], bi[1]);
                        v[2][k] = __builtin_fmaf(o2, sc[2], bi[2]);
                    }
                } else {
#pragma unroll
                    for (int c = 0; c < 3; c++)
#pragma unroll
                        for (int k = 0; k < PX; k++) {
                            float t = v[c][k];
                            // a convex blend of u8 values stays inside [0,255]: rounding alone saturates it
                            if constexpr (QUANT) t = NEAREST ? t : __builtin_rintf(t);
                            if constexpr (NORM) t = __builtin_fmaf(t, sc[c], bi[c]);
                            v[c][k] = t;
                        }
                }
                const int x0 = hf ? (dw - t0 - cnt) : t0;
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, x0, cnt, v, hf);
            }
            wave_sync();  // ring rows of this step may be overwritten from here on

            // ---- commit the next step's rows
            if (has_next) {
                stage_commit(S, lds, lane, new_lo, slot_new, nit, 0, raw);
                for (int first = NL; first < nit; first += NL) {
                    stage_issue(S, lane, new_lo, nit, first, raw);
                    stage_commit(S, lds, lane, new_lo, slot_new, nit, first, raw);
                }
                wave_sync();
                if ((rep_l || rep_r) && lane < nnew) {
                    int sl = slot_new + lane;
                    if (sl >= R) sl -= R;
                    uint32_t *row = lds + sl * pitch;
                    if (rep_l) row[3] = row[4];
                    if (rep_r) row[4 + nc] = row[4 + nc + 1] = row[4 + nc - 1];  // two: under the device edge rule a left tap can lie one beyond
                }
                wave_sync();
                base_slot = base_slot_n;
                a_k = a_n;
                b_k = b_n;
            }
        }
    }
}

// One translation unit per destination type and layout instantiates the kernel (the 48 instantiations in one
// unit took four minutes to compile); RMX_RESIZE_UNIT(T, LAYOUT, name) defines that unit's selector.
template <typename T, int LAYOUT, bool NEAREST>
static KernelFn pick3(bool norm, bool quant, int chain) {
    if constexpr (!NEAREST) {
        if (norm && quant && chain == CHAIN_LINEAR) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, true, false, CHAIN_LINEAR>;
        if (norm && quant && chain == CHAIN_TWIST) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, true, false, CHAIN_TWIST>;
    }
    if (norm && quant) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, true, NEAREST>;
    if (norm) return (KernelFn)rmx_resize_kernel<T, LAYOUT, true, false, NEAREST>;
    return (KernelFn)rmx_resize_kernel<T, LAYOUT, false, false, NEAREST>;
}

#define RMX_RESIZE_UNIT(T, LAYOUT, name)                                              \
    KernelFn name(bool nearest, bool norm, bool quant, int chain) {                   \
        return nearest ? pick3<T, LAYOUT, true>(norm, quant, 0) : pick3<T, LAYOUT, false>(norm, quant, chain); \
    }

}  // namespace rmx
