// K2 fast path: bilinear resize + epilogue for batches in which every written width is a multiple
// of 8 and both batch bases are 16-byte aligned (the training shapes: 224, 256, 384, 640 ...).
//
// One wavefront produces a strip of `aux0` destination rows of one sample, one x-tile at a time:
//   1. the source rows the strip needs are staged ONCE into the wavefront's LDS slice, one dword per
//      pixel (0x..BBGGRR): an item is 4 pixels = 12 source bytes, fetched with one 16-byte load at
//      dword alignment, re-aligned in registers and written with one 16-byte LDS store. All
//      (row, item) pairs of the window form one flat index space dealt to the 64 lanes, and all loads
//      of the window are issued before the first one is consumed, so a wavefront pays one memory
//      round trip per tile and no lane idles on a short row;
//   2. every lane then blends 8 adjacent destination pixels of one row per pass: the two horizontal
//      neighbours of a tap pair are adjacent dwords (aligned LDS reads; reads that are not naturally
//      aligned were measured to be several times slower), unpacked with v_cvt_f32_ubyte*.
//      Coordinates and x weights are computed once per tile, while the loads are in flight;
//   3. quantise / normalise / cast / mirror and 128-bit planar stores, as in the general kernel.
// The arithmetic is the general kernel's, operation for operation. Wavefronts never wait for each
// other; latency is hidden by the other wavefronts resident on the CU (the LDS slice is kept small,
// per sample, by narrowing the x-tile when the source window is large). The kernel is bound by
// vector-ALU issue (about 43 instructions per destination pixel; a wavefront issues one every ~5 cycles
// and a SIMD sustained one every ~6 here), not by memory: instruction count is what every choice above
// minimises. Two variants that were tried and measured slower: taps kept packed and widened inside
// v_fma_mix_f32 (bit-exact through the fp16-subnormal trick, fewer instructions, but each costs more
// issue time), and tighter register budgets for 20-24 wavefronts per CU.
#include "rmx_device.h"
#include "rmx_color_math.h"
#include "rmx_launch.h"

#include <type_traits>

namespace rmx {

extern __shared__ uint32_t rmx_lds_fast[];

RMX_DEV float src_coord_f(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}

constexpr int SB = 12;  // staging slots per lane issued back to back: 12 x 64 items = a 12 KB window

// CHAIN: a colour node between the (quantised) resize and the normalisation, see chain_colour().
template <typename T, int LAYOUT, bool NORM, bool QUANT, int CHAIN>
__global__ void __launch_bounds__(256) rmx_resize_fast_kernel(RmxKArgs a) {
    static_assert(CHAIN == CHAIN_NONE || QUANT, "a colour node in the chain reads the u8 output of the resize node");
    __shared__ __attribute__((aligned(16))) float chain_tables[CHAIN == CHAIN_TWIST ? sizeof(ColorTables) / 4 : 4];
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    // Interleaved fp32 output (96 bytes per lane): the lanes of a row exchange their runs through LDS before storing
    // (store_packed_coalesced); the slab is the tail of the wavefront's LDS slice, the host adds its size to the slice.
    // Measured on the RandomResizedCrop batch: 57.1 -> 48.4 us. Planar fp32 stays within the run-to-run spread (44.7 / 43.8 /
    // 45.9 us) and interleaved fp16 loses more to the larger slice than it gains (35.3 -> 36.2 us): both keep the direct stores.
    constexpr bool COALESCE = sizeof(T) == 4 && LAYOUT == RMX_NHWC;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    // launch geometry comes from the kernel arguments (one scalar load), not from the dispatch packet
    uint32_t wave = xcd_swizzle(blockIdx.x, a.nblocks) * (uint32_t)a.wpb + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, strip;
    wave_to_sample(a, wave, s, strip);
    // the whole 128-byte row at once: one memory round trip before the first use, not one per field group
    // (the empty statement "uses" fields from every part of the row, which keeps the compiler from sinking
    // part of the fetch below the early exit)
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.pc_x), "s"(P.flags), "s"(P.rx), "s"(P.scale[0]), "s"(P.bias[2]), "s"(P.plan[0]));

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
    uint32_t *lds = rmx_lds_fast + (size_t)wib * (a.lds_bytes >> 2);
    uint32_t *slab = COALESCE ? lds + (a.lds_bytes >> 2) - RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>() : nullptr;

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

    // source addressing: dword-aligned base below the sample, 32-bit byte offsets from it
    uint32_t row_stride;
    const uint8_t *simg = sample_base(a, s, row_stride);
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint8_t *base4 = simg - skew;
    const uint64_t left = (uint64_t)((a.src + a.src_bytes) - base4);
    const uint32_t lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;

    // virtual source rows of the strip: a_v .. b_v (clamped into the window when they are fetched)
    const int a_v = (int)floorf(src_coord_f(pcy + r0, ry, offy, fylo));
    const int b_v = (int)floorf(src_coord_f(pcy + r1 - 1, ry, offy, fylo)) + 1;
    const int nrows = b_v - a_v + 1;

    const int tile_w = max(P.plan[0], PX);  // never 0: it is the step of the tile loop
    for (int xt = 0; xt < dw; xt += tile_w) {
        const int tw = min(dw - xt, tile_w);
        const int L = tw / PX;
        const int G = RMX_WAVE / L;
        const int lr = lane / L;
        const int g = lane - lr * L;
        const int t0 = xt + g * PX;
        const bool lane_on = lr < G;

        const int ixmin = (int)floorf(src_coord_f(pcx + xt, rx, offx, fxlo));
        const int ixmax = (int)floorf(src_coord_f(pcx + xt + tw - 1, rx, offx, fxlo));
        const int cs = max(min(ixmin, xhi), xlo);
        const int ce = max(min(ixmax + 1, xhi), xlo);
        const int nc = ce - cs + 1;
        const bool rep_l = ixmin < xlo, rep_r = ixmax + 1 > xhi;
        const int ipr = (nc + 3) >> 2;       // 4-pixel items per row
        const int pitch = 4 + ipr * 4 + 4;   // LDS row in dwords: [pad + left replica][pixels][right replica + pad]
        const uint32_t col0 = (uint32_t)cs * 3u + skew;

        // ---- 1. stage the window
        const int total = nrows * ipr;
        const float inv_ipr = 1.0f / (float)ipr;
        const uint32_t last_off = (uint32_t)max(min(b_v, yhi), ylo) * row_stride + col0;
        const bool safe = (uint64_t)(last_off & ~3u) + 12ull * (uint64_t)ipr + 4ull <= (uint64_t)lim;
        // dword offset of the left neighbour inside an LDS row, and the x weights
        uint32_t offd[PX];
        float wx[PX], omx[PX];
        auto taps = [&]() {
#pragma unroll
            for (int k = 0; k < PX; k++) {
                float sx = src_coord_f(pcx + t0 + k, rx, offx, fxlo);
                float fx = floorf(sx);
                wx[k] = sx - fx;
                omx[k] = 1.0f - wx[k];
                offd[k] = (uint32_t)(4 + ((int)fx - cs));
            }
        };
        // Every load of the window is issued before the first one is consumed, straight-line and
        // unconditional so that the loads stay in flight together (items beyond the window repeat its last
        // item); the tap set-up runs while they are. NS = slots of 64 items.
        auto stage = [&](auto nsc) {
            constexpr int NS = decltype(nsc)::value;
            u32x4_a4 v[NS];
            uint32_t dst_off[NS], ph[NS];
#pragma unroll
            for (int j = 0; j < NS; j++) {
                const int idx = min(j * RMX_WAVE + lane, total - 1);
                // idx / ipr and idx % ipr: (idx + 0.5) / ipr is at least 0.5/ipr away from an integer, far more
                // than the rounding error of the product (idx < 2^16), so the truncation is exact
                const int r = (int)(((float)idx + 0.5f) * inv_ipr);
                const int c = idx - __mul24(r, ipr);
                const int ysrc = max(min(a_v + r, yhi), ylo);
                const uint32_t off = (uint32_t)__mul24(ysrc, (int)row_stride) + col0 + 12u * (uint32_t)c;
                v[j] = *reinterpret_cast<const u32x4_a4 *>(base4 + (off & ~3u));
                dst_off[j] = (uint32_t)(__mul24(r, pitch) + 4 + 4 * c);
                ph[j] = off & 3u;
            }
            taps();
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
            else stage(std::integral_constant<int, SB>{});
            // windows of more than SB*64 items (only with an LDS budget above the default): the rest, batch by batch
            for (int base = SB * RMX_WAVE; base < total; base += RMX_WAVE) {
                const int idx = base + lane;
                if (idx < total) {
                    const int r = idx / ipr;
                    const int c = idx - r * ipr;
                    const int ysrc = max(min(a_v + r, yhi), ylo);
                    const uint32_t off = (uint32_t)ysrc * row_stride + col0 + 12u * (uint32_t)c;
                    const u32x4_a4 q = *reinterpret_cast<const u32x4_a4 *>(base4 + (off & ~3u));
                    const uint32_t d[4] = {q.x, q.y, q.z, q.w};
                    *reinterpret_cast<uint4 *>(lds + r * pitch + 4 + 4 * c) = expand4(d, off & 3u);
                }
            }
        } else {
            // the window touches the last bytes of the batch buffer: byte loads, each one bounds-checked
            taps();
            for (int idx = lane; idx < total; idx += RMX_WAVE) {
                const int r = idx / ipr;
                const int c = idx - r * ipr;
                const int ysrc = max(min(a_v + r, yhi), ylo);
                const uint32_t off = (uint32_t)ysrc * row_stride + col0 + 12u * (uint32_t)c;
                uint32_t px[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t w = 0;
#pragma unroll
                    for (int b = 0; b < 3; b++) {
                        const uint32_t ob = off + 3u * i + b;
                        w |= (ob < lim ? (uint32_t)base4[ob] : 0u) << (8 * b);
                    }
                    px[i] = w;
                }
                *reinterpret_cast<uint4 *>(lds + r * pitch + 4 + 4 * c) = make_uint4(px[0], px[1], px[2], px[3]);
            }
        }
        wave_sync();
        // clamp-to-edge: the pixel next to the window's first / last column repeats it
        if (rep_l || rep_r) {
            for (int rr = lane; rr < nrows; rr += RMX_WAVE) {
                uint32_t *row = lds + rr * pitch;
                if (rep_l) row[3] = row[4];
                if (rep_r) row[4 + nc] = row[4 + nc + 1] = row[4 + nc - 1];  // two: under the device edge rule a left tap can lie one beyond
            }
            wave_sync();
        }

        // ---- 2./3. blend, epilogue, store: G rows per pass
        const int x0 = hf ? (dw - t0 - PX) : t0;
        for (int rs = r0; rs < r1; rs += G) {
            const int r = rs + lr;
            if (lane_on && r < r1) {
                float sy = src_coord_f(pcy + r, ry, offy, fylo);
                float fy = floorf(sy);
                float wy = sy - fy;
                const uint32_t *row0 = lds + ((int)fy - a_v) * pitch;
                const uint32_t *row1 = row0 + pitch;
                const float omy = 1.0f - wy;
                float v[3][PX];
#pragma unroll
                for (int k = 0; k < PX; k++) {
                    const uint32_t tl = row0[offd[k]], tr = row0[offd[k] + 1], bl = row1[offd[k]], br = row1[offd[k] + 1];
                    float w00 = omy * omx[k], w01 = omy * wx[k], w10 = wy * omx[k];
                    float o0 = __builtin_fmaf(ubyte0(tl), w00, __builtin_fmaf(ubyte0(tr), w01, __builtin_fmaf(ubyte0(bl), w10, ubyte0(br) * wy * wx[k])));
                    float o1 = __builtin_fmaf(ubyte1(tl), w00, __builtin_fmaf(ubyte1(tr), w01, __builtin_fmaf(ubyte1(bl), w10, ubyte1(br) * wy * wx[k])));
                    float o2 = __builtin_fmaf(ubyte2(tl), w00, __builtin_fmaf(ubyte2(tr), w01, __builtin_fmaf(ubyte2(bl), w10, ubyte2(br) * wy * wx[k])));
                    // a convex blend of u8 values stays inside [0,255]: rounding alone saturates it
                    if constexpr (QUANT) {
                        o0 = __builtin_rintf(o0); o1 = __builtin_rintf(o1); o2 = __builtin_rintf(o2);
                    }
                    chain_colour<CHAIN>(o0, o1, o2, cp, sh2, sh4, ctab);
                    if constexpr (NORM) {
                        o0 = __builtin_fmaf(o0, sc[0], bi[0]); o1 = __builtin_fmaf(o1, sc[1], bi[1]); o2 = __builtin_fmaf(o2, sc[2], bi[2]);
                    }
                    v[0][k] = o0; v[1][k] = o1; v[2][k] = o2;
                }
                PackedGroup<T> packed;
                pack_group<T, LAYOUT>(v, hf, packed);
                if constexpr (COALESCE) store_packed_coalesced<T, LAYOUT>(slab, lane - g, hf ? (L - 1 - g) : g, L, dimg, a.dst_h, a.dst_w, r, x0, packed);
                else store_packed<T, LAYOUT, sizeof(T) == 2>(dimg, a.dst_h, a.dst_w, r, x0, packed);  // fp16: streaming stores
            }
        }
        if (xt + tile_w < dw) wave_sync();  // the next tile overwrites the LDS slice
    }
}

template <typename T, int LAYOUT>
static KernelFn pick3(bool norm, bool quant, int chain) {
    if (norm && quant && chain == CHAIN_LINEAR) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, true, CHAIN_LINEAR>;
    if (norm && quant && chain == CHAIN_TWIST) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, true, CHAIN_TWIST>;
    if (norm && quant) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, true, CHAIN_NONE>;
    if (norm) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, false, CHAIN_NONE>;
    return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, false, false, CHAIN_NONE>;
}

// chain: 0 none, 1 linear colour node, 2 colour twist between resize and normalisation (only with norm and quant)
KernelFn select_resize_fast_kernel(int dtype, int layout, bool norm, bool quant, int chain, const char **name) {
    *name = "rmx_resize_fast_kernel";
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return pick3<float, RMX_NCHW>(norm, quant, chain);
            case RMX_FP16: return pick3<__half, RMX_NCHW>(norm, quant, chain);
            default: return pick3<uint8_t, RMX_NCHW>(norm, quant, chain);
        }
    }
    switch (dtype) {
        case RMX_FP32: return pick3<float, RMX_NHWC>(norm, quant, chain);
        case RMX_FP16: return pick3<__half, RMX_NHWC>(norm, quant, chain);
        default: return pick3<uint8_t, RMX_NHWC>(norm, quant, chain);
    }
}

}  // namespace rmx
