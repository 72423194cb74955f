// K4: inverse-map affine warp (WarpAffine / Rotate), bilinear or nearest, constant-0 outside
// the source ROI; u8 NHWC in, T/LAYOUT out.
//
// A wavefront owns a destination tile of 32 columns x (16 x passes) rows. The tile's corners are pushed
// through the affine map to get the source bounding box (every pixel of the tile maps inside it: each
// step of the coordinate law is monotone in x and in y, also after rounding), which is staged into the
// wavefront's LDS slice, one dword per pixel, with all loads of the box in flight together; one extra
// column and row repeat the ROI's last column / row, so the right and lower neighbours of a tap are always
// at +1 and +pitch. Each lane then produces 8 adjacent destination pixels of one row per pass, branch-free:
// taps of pixels that fall outside the ROI are read from wherever their (meaningless) address points inside
// the slice and the result is replaced by 0. When the box does not fit the slice (strong minification) the
// wavefront gathers from global memory instead.
//
// RAW (every source row starts at the same byte phase: row strides multiples of 4): the box travels from global memory
// straight into LDS as packed bytes (global_load_lds_dwordx4, 16 bytes per lane: no vector register, no unpacking, no LDS
// store; piece i of the box, rows one after the other, is loaded by lane i & 63 of load instruction i >> 6), three bytes
// per pixel instead of four, and a tap pair (two packed pixels, 6 bytes at any byte phase) is read as three aligned dwords
// and realigned with two v_alignbyte. Values and operations from there on are the same.
#include "rmx_device.h"
#include "rmx_launch.h"

#include <type_traits>

#ifndef RMX_WARP_NT
#define RMX_WARP_NT false
#endif

namespace rmx {

extern __shared__ uint32_t rmx_lds_warp[];
typedef __attribute__((address_space(3))) uint32_t lds_u32;  // explicit LDS pointers: 32-bit address arithmetic

constexpr int WTW = 32, WTH = 16;  // destination tile: 4 lanes x 8 px wide, 16 rows per pass
constexpr int WFP = 60;            // fixed LDS pitch (dwords) of boxes that fit it
constexpr int WRP = kWarpRawPieces;  // RAW: fixed LDS pitch in 16-byte pieces (an odd number spreads the rows over the LDS banks)

RMX_DEV uint32_t load_px_global(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16);
}

// floor(x) as an integer in one instruction (saturating; 0 for NaN)
RMX_DEV int floor_i32(float x) {
    int r;
    asm("v_cvt_flr_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

template <typename T, int LAYOUT, bool NEAREST, bool RAW>
__global__ void __launch_bounds__(256) rmx_warp_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, a.nblocks) * (uint32_t)a.wpb + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, tile;
    wave_to_sample(a, wave, s, tile);
    const int tiles_x = a.aux0;
    const int passes = a.aux1 >> 8;
    const bool packed_ok = (a.aux1 & 1) != 0;
    const int ty = tile / tiles_x, tx = tile - ty * tiles_x;
    // the whole table row in one round trip
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.flags), "s"(P.m[0]), "s"(P.m[5]));
    const int dw = P.dst_w, dh = P.dst_h;
    const int X0 = tx * WTW, Y0 = ty * (WTH * passes);
    if (X0 >= dw || Y0 >= dh) return;

    const int xlo = P.src_x, ylo = P.src_y;
    const int xhi = xlo + P.src_w - 1, yhi = ylo + P.src_h - 1;
    const float m0 = P.m[0], m1 = P.m[1], m2 = P.m[2], m3 = P.m[3], m4 = P.m[4], m5 = P.m[5];
    const float dcx = (float)(dw >> 1), dcy = (float)(dh >> 1);
    const float scx = (float)(xlo + (P.src_w >> 1)), scy = (float)(ylo + (P.src_h >> 1));

    uint32_t row_stride;
    const uint8_t *simg = sample_base(a, s, row_stride);
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *lds = rmx_lds_warp + (size_t)wib * (a.lds_bytes >> 2);

    // source bounding box of the tile (wave-uniform), one pixel of margin, clipped to the ROI
    const int X1 = min(X0 + WTW, dw) - 1, Y1 = min(Y0 + WTH * passes, dh) - 1;
    float bxmin = 3.0e38f, bxmax = -3.0e38f, bymin = 3.0e38f, bymax = -3.0e38f;
    bool corners_ok = true;
#pragma unroll
    for (int cy = 0; cy < 2; cy++)
#pragma unroll
        for (int cx = 0; cx < 2; cx++) {
            float xr = (float)(cx ? X1 : X0) - dcx, yr = (float)(cy ? Y1 : Y0) - dcy;
            float sx = __builtin_fmaf(xr, m0, __builtin_fmaf(yr, m1, m2)) + scx;
            float sy = __builtin_fmaf(xr, m3, __builtin_fmaf(yr, m4, m5)) + scy;
            if constexpr (NEAREST) {
                sx += 0.5f;
                sy += 0.5f;
            }
            bxmin = __builtin_fminf(bxmin, sx); bxmax = __builtin_fmaxf(bxmax, sx);
            bymin = __builtin_fminf(bymin, sy); bymax = __builtin_fmaxf(bymax, sy);
            corners_ok = corners_ok && sx == sx && sy == sy;
        }
    // every pixel of the tile maps between the corner extremes: when those lie inside the ROI no pixel needs a test
    const bool all_in = corners_ok && bxmin >= (float)xlo && bymin >= (float)ylo && bxmax < (float)(xhi + 1) && bymax < (float)(yhi + 1);
    // keep the float->int conversions in range for degenerate matrices
    bxmin = __builtin_fmaxf(bxmin, -1.0e6f); bxmax = __builtin_fminf(bxmax, 1.0e6f);
    bymin = __builtin_fmaxf(bymin, -1.0e6f); bymax = __builtin_fminf(bymax, 1.0e6f);
    const int bx0 = max((int)floorf(bxmin) - 1, xlo), bx1 = min((int)floorf(bxmax) + 2, xhi);
    const int by0 = max((int)floorf(bymin) - 1, ylo), by1 = min((int)floorf(bymax) + 2, yhi);
    const int bw = bx1 - bx0 + 1, bh = by1 - by0 + 1;
    const bool empty = bw <= 0 || bh <= 0;
    // staged box: bw columns + the repeated last one, bh rows + the repeated last one
    const int items = (max(bw, 0) + 1 + 3) >> 2;
    // Boxes of at most WFP - 1 columns (every tile of a map that does not minify) are staged at ONE pitch, known to the
    // compiler: the address of a tap is two instructions (a 24-bit multiply-add and a shift-add) and the row below is an
    // offset inside the read instruction. 15 items: an odd number of 16-byte items spreads the rows over the LDS banks.
    // RAW: a row is ppr 16-byte pieces from the dword that holds pixel bx0 (byte phase ph inside it)
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint32_t colb = (uint32_t)max(bx0, 0) * 3u + skew;
    const int ph = (int)(colb & 3u);
    const int ppr_box = (ph + 3 * (max(bw, 0) + 1) + 15) >> 4;
    const bool fixed = RAW ? ppr_box <= WRP : items * 4 <= WFP;
    const int ppr = fixed ? WRP : ppr_box;
    const int pitch = RAW ? ppr * 4 : (fixed ? WFP : items * 4);  // dwords
    const int total = (bh + 1) * (RAW ? ppr : items);            // 16-byte pieces (RAW) or four-pixel items of the box
    // (RAW: the three dwords read for the last tap of the last row may reach 8 bytes behind the box)
    const bool use_lds = !empty && total <= 16 * RMX_WAVE && (size_t)(bh + 1) * pitch * 4 + (RAW ? 16 : 0) <= (size_t)a.lds_bytes;

    const int lr = lane >> 2, g = lane & 3;
    const int x0 = X0 + g * PX;
    const int cnt = min(PX, dw - x0);
    const float xr0 = (float)x0 - dcx;

    if (empty) {
        // every pixel of the tile maps outside the ROI: the fill value
        float z[3][PX];
#pragma unroll
        for (int c = 0; c < 3; c++)
#pragma unroll
            for (int k = 0; k < PX; k++) z[c][k] = 0.0f;
        for (int pass = 0; pass < passes; pass++) {
            const int y = Y0 + pass * WTH + lr;
            if (y < dh && cnt > 0) store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, y, x0, cnt, z, false);
        }
        return;
    }
    if (!use_lds) {
        // a box too large for the slice: per-pixel gathers from global memory
        for (int pass = 0; pass < passes; pass++) {
            const int y = Y0 + pass * WTH + lr;
            if (y >= dh || cnt <= 0) continue;
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
                    const uint32_t tl = load_px_global(simg + (size_t)iy0 * row_stride + (size_t)ix0 * 3);
                    if constexpr (NEAREST) {
                        o0 = ubyte0(tl); o1 = ubyte1(tl); o2 = ubyte2(tl);
                    } else {
                        const uint32_t tr = load_px_global(simg + (size_t)iy0 * row_stride + (size_t)ix1 * 3);
                        const uint32_t bl = load_px_global(simg + (size_t)iy1 * row_stride + (size_t)ix0 * 3);
                        const uint32_t br = load_px_global(simg + (size_t)iy1 * row_stride + (size_t)ix1 * 3);
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
            store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, y, x0, cnt, v, false);
        }
        return;
    }

    if constexpr (RAW) {
        // ---- the box straight into LDS: piece idx = (row, piece of the row) in row order lands at byte 16 idx of the slice
        const uint8_t *base4 = simg - skew;
        const uint32_t col4 = colb & ~3u;
        lds_u8 *ldsb = (lds_u8 *)(lds_ptr_t)rmx_lds_warp + (uint32_t)to_sgpr((int)((uint32_t)wib * (uint32_t)a.lds_bytes));
        // every piece of the box lies inside the batch buffer (the last rows of the last sample may not)
        const bool safe = simg + ((size_t)min(by1 + 1, yhi) * row_stride + (size_t)bx0 * 3 + 16 * (size_t)ppr) <= buf_end;
        const float inv_ppr = 1.0f / (float)ppr;
        if (safe) {
            for (int j0 = 0; j0 < total; j0 += RMX_WAVE) {
                const int idx = j0 + lane;
                // idx / ppr: (idx + 0.5) / ppr is at least 0.5/ppr away from an integer, so the truncation is exact
                const int r = fixed ? idx / WRP : (int)(((float)idx + 0.5f) * inv_ppr);
                const int c = idx - __mul24(r, ppr);
                const uint32_t off = (uint32_t)min(by0 + r, yhi) * row_stride + col4 + 16u * (uint32_t)c;
                if (idx < total) __builtin_amdgcn_global_load_lds((glb_ptr_t)(base4 + off), (lds_ptr_t)(ldsb + 16 * j0), 16, 0, RMX_LDS_LOAD_AUX);
            }
            // the compiler does not order LDS reads behind loads into LDS: await them explicitly
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            // the box touches the last bytes of the batch buffer: bounds-checked byte loads, stored by the lanes
            const uint64_t left = (uint64_t)(buf_end - base4);
            const uint32_t lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;
            for (int idx = lane; idx < total; idx += RMX_WAVE) {
                const int r = idx / ppr, c = idx - r * ppr;
                const uint32_t off = (uint32_t)min(by0 + r, yhi) * row_stride + col4 + 16u * (uint32_t)c;
                lds_u32 *dst4 = (lds_u32 *)(ldsb + 16 * idx);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t v = 0;
#pragma unroll
                    for (int b = 0; b < 4; b++) {
                        const uint32_t ob = off + 4u * i + b;
                        v |= (ob < lim ? (uint32_t)base4[ob] : 0u) << (8 * b);
                    }
                    dst4[i] = v;
                }
            }
        }
        wave_sync();
        // the column behind the box repeats its last column where that is the ROI's last column (only then is it read)
        if (bx1 == xhi) {
            for (int r = lane; r <= bh; r += RMX_WAVE) {
                lds_u8 *px = ldsb + r * (pitch * 4) + ph + 3 * (bw - 1);
                px[3] = px[0];
                px[4] = px[1];
                px[5] = px[2];
            }
            wave_sync();
        }
    } else
    // ---- stage the box: (row, 4-pixel item) pairs form one flat index space dealt to the lanes; rows beyond
    // the box repeat the ROI's last row (the clamp does it); all loads go out before the first is consumed
    {
        const uint8_t *base4 = simg - skew;
        const uint32_t col0 = (uint32_t)bx0 * 3u + skew;
        const float inv_items = 1.0f / (float)items;
        // the last load of the box stays inside the batch buffer
        const bool safe = simg + ((size_t)min(by1 + 1, yhi) * row_stride + (size_t)bx0 * 3 + 12 * (size_t)items + 4) <= buf_end;
        auto stage = [&](auto nsc) {
            constexpr int NS = decltype(nsc)::value;
            u32x4_a4 v[NS];
            uint32_t dst_off[NS], ph[NS];
#pragma unroll
            for (int j = 0; j < NS; j++) {
                const int idx = min(j * RMX_WAVE + lane, total - 1);
                // idx / items: (idx + 0.5) / items is at least 0.5/items away from an integer, so the truncation is exact
                const int r = (int)(((float)idx + 0.5f) * inv_items);
                const int c = idx - __mul24(r, items);
                const int ysrc = min(by0 + r, yhi);
                const uint32_t off = (uint32_t)ysrc * row_stride + col0 + 12u * (uint32_t)c;
                v[j] = *reinterpret_cast<const u32x4_a4 *>(base4 + (off & ~3u));
                dst_off[j] = (uint32_t)(__mul24(r, pitch) + 4 * c);
                ph[j] = off & 3u;
            }
#pragma unroll
            for (int j = 0; j < NS; j++) {
                const uint32_t d[4] = {v[j].x, v[j].y, v[j].z, v[j].w};
                const uint4 px = expand4(d, ph[j]);
                if (j * RMX_WAVE + lane < total) *reinterpret_cast<uint4 *>(lds + dst_off[j]) = px;
            }
        };
        if (safe) {
            if (total <= 4 * RMX_WAVE) stage(std::integral_constant<int, 4>{});
            else if (total <= 8 * RMX_WAVE) stage(std::integral_constant<int, 8>{});
            else stage(std::integral_constant<int, 16>{});
        } else {
            // the box touches the last bytes of the batch buffer: bounds-checked loads
            for (int idx = lane; idx < total; idx += RMX_WAVE) {
                const int r = idx / items, c = idx - r * items;
                const uint8_t *p = simg + (size_t)min(by0 + r, yhi) * row_stride + (size_t)(bx0 + 4 * c) * 3;
                uint32_t w[3];
                load_realigned<4>(p, buf_end, w);
                uint4 px;
                px.x = w[0];
                px.y = __builtin_amdgcn_alignbyte(w[1], w[0], 3);
                px.z = __builtin_amdgcn_alignbyte(w[2], w[1], 2);
                px.w = w[2] >> 8;
                *reinterpret_cast<uint4 *>(lds + r * pitch + 4 * c) = px;
            }
        }
        wave_sync();
        // the column behind the box repeats its last column (it is read only when that is the ROI's last column)
        for (int r = lane; r <= bh; r += RMX_WAVE) lds[r * pitch + bw] = lds[r * pitch + bw - 1];
        wave_sync();
    }

    // ---- gather and blend, branch-free
    // LDS byte address of source pixel (0, 0): the slice's base minus the box origin (may lie below the slice)
    // (RAW: byte address of the first byte of source pixel (0, 0), three bytes per pixel)
    const int lbase0 = RAW ? (int)(uint32_t)(uintptr_t)(lds_u32 *)lds + ph - (4 * by0 * pitch + 3 * bx0)
                           : (int)(uint32_t)(uintptr_t)(lds_u32 *)lds - 4 * (by0 * pitch + bx0);
    // pixels whose floor lies inside the ROI: xlo <= s < xhi + 1 (and not NaN), tested on the clamped coordinate
    // (upper bounds: the float just below xhi + 1, a positive number, so one step down in its bit pattern)
    const float cx_lo = (float)xlo, cx_hi = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, (float)(xhi + 1)) - 1u);
    const float cy_lo = (float)ylo, cy_hi = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, (float)(yhi + 1)) - 1u);
    int lbase_v = lbase0;  // the same in a vector register: the multiply-add takes only one scalar operand
    asm volatile("" : "+v"(lbase_v));
    auto gather = [&](auto chk, auto fix) {
        constexpr bool CHECK = decltype(chk)::value;
        constexpr bool FIXED = decltype(fix)::value;
        for (int pass = 0; pass < passes; pass++) {
            const int y = Y0 + pass * WTH + lr;
            if (y >= dh || cnt <= 0) continue;
            const float yr = (float)y - dcy;
            const float cxy = __builtin_fmaf(yr, m1, m2), cyy = __builtin_fmaf(yr, m4, m5);
            float v[3][PX];
            // A pixel in two steps: fetch (coordinates, tap address, the LDS reads of its taps) and blend. The reads of pixel
            // k + 1 are issued before pixel k is blended, so that a wavefront waits for LDS once per row instead of once per
            // pixel (left to the compiler's order, every pixel's reads were followed at once by the wait for them): 65.6 -> 64.1 us
            // on 128 images of 512 x 512.
            typedef uint32_t u32x2_r __attribute__((ext_vector_type(2)));
            struct Taps {
                u32x2_r top, bot;  // the first two dwords of the upper and of the lower row (RAW), or the two pixels of each row
                uint32_t t2, b2;   // RAW: the third dword of each row
                float sx, sy;
                uint32_t tph;
                bool inb;
            };
            // RAW bilinear taps at the fixed pitch: the reads are written out (one address register for both rows, the row
            // below at an offset inside the instruction) and awaited by a count, so that the reads of the next pixel stay in
            // flight while this one is blended; the compiler's own bookkeeping would wait for every outstanding read.
            constexpr bool BY_HAND = RAW && FIXED && !NEAREST;
            auto fetch = [&](int k) {
                Taps t;
                const float xr = xr0 + (float)k;  // == (float)(x0 + k) - dcx: small integers, exact
                float sx = __builtin_fmaf(xr, m0, cxy) + scx;
                float sy = __builtin_fmaf(xr, m3, cyy) + scy;
                if constexpr (NEAREST) {
                    sx += 0.5f;
                    sy += 0.5f;
                }
                t.inb = true;
                if constexpr (CHECK) {
                    // Clamped into the ROI (a NaN becomes the lower bound): equal to the coordinate exactly when the pixel is
                    // inside, and an address inside the staged box also when it is not (the box holds the ROI's border
                    // wherever the tile reaches beyond it).
                    const float qx = __builtin_fminf(__builtin_fmaxf(sx, cx_lo), cx_hi);
                    const float qy = __builtin_fminf(__builtin_fmaxf(sy, cy_lo), cy_hi);
                    t.inb = qx == sx && qy == sy;
                    sx = qx;
                    sy = qy;
                }
                t.sx = sx;
                t.sy = sy;
                const int ix0 = floor_i32(sx), iy0 = floor_i32(sy);
                const lds_u32 *t0p, *t1p;
                t.tph = 0;  // RAW: byte phase of the tap pair inside its first dword
                if constexpr (RAW) {
                    uint32_t rowb, adr;
                    if constexpr (FIXED) asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(rowb) : "v"(iy0), "s"(WRP * 16), "v"(lbase_v));
                    else rowb = (uint32_t)(__mul24(iy0, pitch * 4) + lbase0);
                    asm("v_mad_i32_i24 %0, %1, 3, %2" : "=v"(adr) : "v"(ix0), "v"(rowb));
                    t.tph = adr & 3u;
                    t0p = (const lds_u32 *)(adr & ~3u);
                    t1p = FIXED ? t0p + WRP * 4 : t0p + pitch;
                } else if constexpr (FIXED) {
                    // byte address: a 24-bit multiply-add of the row onto the (scalar) slice base, a shift-add of the column
                    // (spelled out: left to itself the compiler makes a shift, a multiply and a three-way add of it)
                    uint32_t rowb, adr;
                    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(rowb) : "v"(iy0), "s"(WFP * 4), "v"(lbase_v));
                    asm("v_lshl_add_u32 %0, %1, 2, %2" : "=v"(adr) : "v"(ix0), "v"(rowb));
                    t0p = (const lds_u32 *)adr;
                    t1p = t0p + WFP;
                } else {
                    t0p = (const lds_u32 *)(uint32_t)(((uint32_t)(__mul24(iy0, pitch) + ix0) << 2) + (uint32_t)lbase0);
                    t1p = t0p + pitch;
                }
                if constexpr (BY_HAND) {
                    static_assert(WRP * 4 + 2 < 256, "the row below must be reachable by the 8-bit dword offsets of ds_read2_b32");
                    // (the values are taken apart only behind the wait: nothing may copy a register before its data has arrived)
                    asm volatile("ds_read2_b32 %0, %4 offset1:1\n\tds_read_b32 %1, %4 offset:8\n\t"
                                 "ds_read2_b32 %2, %4 offset0:%5 offset1:%6\n\tds_read_b32 %3, %4 offset:%7"
                                 : "=&v"(t.top), "=&v"(t.t2), "=&v"(t.bot), "=&v"(t.b2)
                                 : "v"((uint32_t)(uintptr_t)t0p), "n"(WRP * 4), "n"(WRP * 4 + 1), "n"(WRP * 16 + 8));
                    return t;
                }
                t.top = (u32x2_r){t0p[0], 0u};
                t.bot = (u32x2_r){0u, 0u};
                t.t2 = t.b2 = 0u;
                if constexpr (RAW) t.top.y = t0p[1];
                if constexpr (!NEAREST) {
                    t.top.y = t0p[1];
                    t.bot = (u32x2_r){t1p[0], t1p[1]};
                    if constexpr (RAW) {
                        t.t2 = t0p[2];
                        t.b2 = t1p[2];
                    }
                }
                return t;
            };
            // BY_HAND: the taps of a pixel have arrived when at most `behind` younger read instructions are outstanding
            // (LDS operations of a wavefront complete in issue order); everything that reads the taps comes behind this.
            auto arrived = [&](Taps &t, auto behind) {
                if constexpr (BY_HAND)
                    asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(t.top), "+v"(t.t2), "+v"(t.bot), "+v"(t.b2) : "n"(decltype(behind)::value));
            };
            auto blend = [&](int k, const Taps &tp) {
                struct { uint32_t tl, tr, t2, bl, br, b2; float sx, sy; uint32_t tph; bool inb; } t = {tp.top.x, tp.top.y, tp.t2, tp.bot.x, tp.bot.y, tp.b2, tp.sx, tp.sy, tp.tph, tp.inb};
                float o0, o1, o2;
                if constexpr (NEAREST) {
                    uint32_t tl = t.tl;
                    if constexpr (RAW) tl = __builtin_amdgcn_alignbyte(t.tr, tl, t.tph);
                    o0 = ubyte0(tl); o1 = ubyte1(tl); o2 = ubyte2(tl);
                } else {
                    // s - floor(s): exact for the non-negative coordinates of pixels inside the ROI
                    const float wx = __builtin_amdgcn_fractf(t.sx), wy = __builtin_amdgcn_fractf(t.sy);
                    const float omx = 1.0f - wx, omy = 1.0f - wy;
                    const float w00 = omy * omx, w01 = omy * wx, w10 = wy * omx;
                    if constexpr (RAW) {
                        // six bytes from byte tph on: TL in bytes 0..2 of the first realigned dword, TR from its byte 3 on
                        const uint32_t tlo = __builtin_amdgcn_alignbyte(t.tr, t.tl, t.tph), thi = __builtin_amdgcn_alignbyte(t.t2, t.tr, t.tph);
                        const uint32_t blo = __builtin_amdgcn_alignbyte(t.br, t.bl, t.tph), bhi = __builtin_amdgcn_alignbyte(t.b2, t.br, t.tph);
                        o0 = __builtin_fmaf(ubyte0(tlo), w00, __builtin_fmaf(ubyte3(tlo), w01, __builtin_fmaf(ubyte0(blo), w10, ubyte3(blo) * wy * wx)));
                        o1 = __builtin_fmaf(ubyte1(tlo), w00, __builtin_fmaf(ubyte0(thi), w01, __builtin_fmaf(ubyte1(blo), w10, ubyte0(bhi) * wy * wx)));
                        o2 = __builtin_fmaf(ubyte2(tlo), w00, __builtin_fmaf(ubyte1(thi), w01, __builtin_fmaf(ubyte2(blo), w10, ubyte1(bhi) * wy * wx)));
                    } else {
                        o0 = __builtin_fmaf(ubyte0(t.tl), w00, __builtin_fmaf(ubyte0(t.tr), w01, __builtin_fmaf(ubyte0(t.bl), w10, ubyte0(t.br) * wy * wx)));
                        o1 = __builtin_fmaf(ubyte1(t.tl), w00, __builtin_fmaf(ubyte1(t.tr), w01, __builtin_fmaf(ubyte1(t.bl), w10, ubyte1(t.br) * wy * wx)));
                        o2 = __builtin_fmaf(ubyte2(t.tl), w00, __builtin_fmaf(ubyte2(t.tr), w01, __builtin_fmaf(ubyte2(t.bl), w10, ubyte2(t.br) * wy * wx)));
                    }
                }
                v[0][k] = t.inb ? o0 : 0.0f;
                v[1][k] = t.inb ? o1 : 0.0f;
                v[2][k] = t.inb ? o2 : 0.0f;
            };
            // (one pixel ahead; two ahead, with eight reads outstanding, measured the same: 64.1 us on 128 images of 512 x 512)
            Taps cur = fetch(0);
#pragma unroll
            for (int k = 0; k < PX; k++) {
                Taps nxt = cur;
                if (k + 1 < PX) {
                    nxt = fetch(k + 1);
                    arrived(cur, std::integral_constant<int, 4>{});  // (the four read instructions of the next pixel may be outstanding)
                    __builtin_amdgcn_sched_barrier(0);               // (the next pixel's reads stay in front of this pixel's arithmetic)
                } else {
                    arrived(cur, std::integral_constant<int, 0>{});
                }
                blend(k, cur);
                cur = nxt;
            }
            // whole group into 16-byte aligned destination rows: packed stores (the host sets the flag when every
            // written width and the padded width are multiples of 8 and the destination base is 16-byte aligned)
            if (packed_ok && cnt == PX) {
                PackedGroup<T> packed;
                pack_group_dir<T, LAYOUT, false>(v, packed);
                store_packed<T, LAYOUT, RMX_WARP_NT>(dimg, a.dst_h, a.dst_w, y, x0, packed);
            } else {
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, y, x0, cnt, v, false);
            }
        }
    };
    if (fixed) {
        if (all_in) gather(std::false_type{}, std::true_type{});
        else gather(std::true_type{}, std::true_type{});
    } else {
        if (all_in) gather(std::false_type{}, std::false_type{});
        else gather(std::true_type{}, std::false_type{});
    }
}

template <bool NEAREST, bool RAW>
static KernelFn pick(int dtype, int layout) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return (KernelFn)rmx_warp_kernel<float, RMX_NCHW, NEAREST, RAW>;
            case RMX_FP16: return (KernelFn)rmx_warp_kernel<__half, RMX_NCHW, NEAREST, RAW>;
            default: return (KernelFn)rmx_warp_kernel<uint8_t, RMX_NCHW, NEAREST, RAW>;
        }
    }
    switch (dtype) {
        case RMX_FP32: return (KernelFn)rmx_warp_kernel<float, RMX_NHWC, NEAREST, RAW>;
        case RMX_FP16: return (KernelFn)rmx_warp_kernel<__half, RMX_NHWC, NEAREST, RAW>;
        default: return (KernelFn)rmx_warp_kernel<uint8_t, RMX_NHWC, NEAREST, RAW>;
    }
}

// raw: the box as packed bytes, loaded straight into LDS (every source row must start at the same byte phase)
KernelFn select_warp_kernel(int interp, int dtype, int layout, bool raw, const char **name) {
    *name = raw ? "rmx_warp_kernel(raw)" : "rmx_warp_kernel";
    if (raw) return interp == RMX_INTERP_NEAREST ? pick<true, true>(dtype, layout) : pick<false, true>(dtype, layout);
    return interp == RMX_INTERP_NEAREST ? pick<true, false>(dtype, layout) : pick<false, false>(dtype, layout);
}

}  // namespace rmx
