// K2 streaming path: bilinear resize + epilogue for batches in which every source row starts at the same byte phase (row
// stride a multiple of 4: padded batches whose width is a multiple of 4, which the training shapes are). Two forms:
//   ALIGNED  every written width a multiple of 8 and a 16-byte aligned destination base: a lane's 8 pixels leave as packed
//            16-byte stores, held back behind the next window's loads (point 3 below);
//   any      every other width or base (225, 299, 300 ... wide outputs): the same loads, taps, blend and held-back stores;
//            the stores are 16-byte stores at the element's alignment, and the short last group of a row is moved left until
//            it is whole. 35 us against 76 us of the general kernel for 256 images to 225 x 225 fp16.
//
// One wavefront = a strip of destination rows of one sample, one x-tile at a time, as in the staged kernel
// (rmx_kernels_resize_fast.hip), but the source window travels from global memory straight into LDS
// (global_load_lds_dwordx4: 16 bytes per lane, no vector register, no unpacking, no LDS store instruction):
//   1. LDS holds the raw packed-RGB rows. A row is a sequence of 16-byte pieces: piece 0 is a margin for the left
//      edge replica, pieces 1.. are the row's bytes from the dword that holds the window's first pixel. One load
//      instruction per source row and 64 pieces; the row's address and LDS slot are scalar arithmetic. The compiler
//      does not order LDS reads behind such loads, so arrival is awaited with an explicit s_waitcnt between two
//      wavefront fences; the x taps of a tile are computed while its first window's loads are in flight;
//   2. the blend reads a tap pair (two packed pixels, 6 bytes at any byte phase) as three aligned dwords and
//      realigns them with two v_alignbyte; every value and every operation after that is the general kernel's,
//      operation for operation (bit-identical results);
//   3. the stores of a window's last pass wait in registers until the next window's loads have been started, so that
//      the wait for those loads (operations of a wavefront complete in issue order) never waits for a store.
// Against the staged kernel this trades about 25 staging instructions per 4 source pixels for 4 realignments per
// destination pixel, frees the registers the staged loads occupy and needs a quarter less LDS (3 bytes per pixel
// instead of 4). Measured on the RandomResizedCrop batch (256 images to 224 x 224 fp16) with every launch reading and
// writing buffers that were not touched for a gigabyte: 32.1 us against 36.4 us; replayed on one cache-resident pair
// 26.3 against 29.4 us. Tried and measured slower: two LDS windows per wavefront with the next window's loads in flight
// during the blend (38-41 us: 12 KB of LDS per wavefront leaves 13 wavefronts per CU), all LDS reads of a pass issued
// before its arithmetic (129 registers, 3 wavefronts per SIMD), register budgets of 96 and 80 (spills), several windows
// below each other per wavefront (fewer instructions, but too few wavefronts to fill the chip evenly).
#include "rmx_device.h"
#include "rmx_color_math.h"
#include "rmx_launch.h"

#include <type_traits>

#ifndef RMX_DMA_NT
#define RMX_DMA_NT (sizeof(T) == 2)  // fp16: streaming stores
#endif
// Measurement builds only (results are wrong): bit 0 leaves out the loads of the source window, bit 1 the stores of the
// result, bit 2 the blend (one LDS read per row, no arithmetic: the kernel's memory traffic with next to no instructions),
// so that a timing shows what each part costs by itself. 0 in the library.
#ifndef RMX_DMA_EXPERIMENT
#define RMX_DMA_EXPERIMENT 0
#endif

namespace rmx {

extern __shared__ uint32_t rmx_lds_dma[];

// (measurement builds: every word of a group that is not stored still has to be computed)
template <typename T>
RMX_DEV void keep_alive(const PackedGroup<T> &g) {
#pragma unroll
    for (int i = 0; i < PackedGroup<T>::WORDS; i++) asm volatile("" ::"v"(g.w[i]));
}

RMX_DEV float src_coord_d(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}


// One x-tile of a wavefront's rows: destination columns [xt, xt + tw) and the source columns they read. Wave-uniform.
struct DmaTile {
    int xt, tw;
    int cs, nc;      // source columns cs .. cs + nc - 1
    int ph;          // byte phase of pixel cs inside its dword
    int ppr;         // 16-byte pieces per LDS row (margin + data + room for the right replicas)
    int nd;          // data pieces per row
    uint32_t col4;   // byte offset (from base4) of the dword that holds pixel cs, within a row
    bool rep_l, rep_r;
};

// CHAIN: a colour node between the (quantised) resize and the normalisation, see chain_colour().
// ALIGNED: every written width is a multiple of 8 and the destination base is 16-byte aligned (whole groups, packed 16-byte
// stores, stores held back); otherwise any width and any base: groups are stored at the alignment of an element, and only a
// tile narrower than 8 pixels has a partial group, stored element by element.
template <typename T, int LAYOUT, bool NORM, bool QUANT, int CHAIN, bool ALIGNED>
__global__ void __launch_bounds__(256) rmx_resize_dma_kernel(RmxKArgs a) {
    static_assert(CHAIN == CHAIN_NONE || QUANT, "a colour node in the chain reads the u8 output of the resize node");
    static_assert(!(ALIGNED && sizeof(T) == 4 && LAYOUT == RMX_NHWC), "interleaved fp32 goes through the coalescing stores of the staged kernel");
    __shared__ __attribute__((aligned(16))) float chain_tables[CHAIN == CHAIN_TWIST ? sizeof(ColorTables) / 4 : 4];
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, a.nblocks) * (uint32_t)a.wpb + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, grp;
    wave_to_sample(a, wave, s, grp);
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.pc_x), "s"(P.flags), "s"(P.rx), "s"(P.scale[0]), "s"(P.bias[2]), "s"(P.plan[1]));

    const int dw = P.dst_w, dh = P.dst_h;
    const int wrows = a.aux0;                        // destination rows of one window
    const int r_begin = grp * wrows * max(a.aux1, 1);  // this wavefront: max(aux1, 1) windows below each other
    if (r_begin >= dh || dw <= 0) return;
    const int r_end = min(r_begin + wrows * max(a.aux1, 1), dh);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;

    const int xlo = P.src_x, ylo = P.src_y;
    const int edge = (int)((P.flags / RMX_S_EDGE_REF) & 1u);
    const int xhi = max(xlo + P.src_w - 1 - edge, xlo), yhi = max(ylo + P.src_h - 1 - edge, ylo);
    const float rx = P.rx, ry = P.ry;
    const float offx = (rx - 1.0f) * 0.5f, offy = (ry - 1.0f) * 0.5f;
    const float fxlo = (float)xlo, fylo = (float)ylo;
    const int pcx = P.pc_x, pcy = P.pc_y;

    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    // (the wavefront's index inside its workgroup comes from a lane id: wave-uniform, but only a scalar register says so)
    const uint32_t slice_off = (uint32_t)to_sgpr((int)((uint32_t)wib * (uint32_t)a.lds_bytes));
    lds_u8 *bufb = (lds_u8 *)(lds_ptr_t)rmx_lds_dma + slice_off;

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }
    const float cp[4] = {P.m[0], P.m[1], P.m[2], P.m[3]};
    const float sh2 = cp[2] + 2.0f, sh4 = cp[2] + 4.0f;
    const ColorTables *ctab = reinterpret_cast<const ColorTables *>(chain_tables);
    if constexpr (CHAIN == CHAIN_TWIST) color_tables_fill(reinterpret_cast<ColorTables *>(chain_tables), lane);

    uint32_t row_stride_v;
    const uint8_t *simg_v = sample_base(a, s, row_stride_v);
    const uint32_t row_stride = (uint32_t)to_sgpr((int)row_stride_v);
    const uint8_t *simg = reinterpret_cast<const uint8_t *>(((uint64_t)(uint32_t)to_sgpr((int)((uintptr_t)simg_v >> 32)) << 32) |
                                                            (uint32_t)to_sgpr((int)(uint32_t)(uintptr_t)simg_v));
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint8_t *base4 = simg - skew;
    const uint64_t left = (uint64_t)((a.src + a.src_bytes) - base4);
    const uint32_t lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;

    const int tile_w = max(P.plan[1], PX);  // never 0: it is the step of the tile loop
    const int ntx = (dw + tile_w - 1) / tile_w;

    // ---- geometry of an x-tile and of a window of it (all wave-uniform)
    auto tile_geom = [&](int tile) {
        DmaTile g;
        g.xt = tile * tile_w;
        g.tw = min(dw - g.xt, tile_w);
        const int ixmin = to_sgpr((int)floorf(src_coord_d(pcx + g.xt, rx, offx, fxlo)));
        const int ixmax = to_sgpr((int)floorf(src_coord_d(pcx + g.xt + g.tw - 1, rx, offx, fxlo)));
        g.cs = max(min(ixmin, xhi), xlo);
        g.nc = max(min(ixmax + 1, xhi), xlo) - g.cs + 1;
        g.rep_l = ixmin < xlo;
        g.rep_r = ixmax + 1 > xhi;
        const uint32_t colb = (uint32_t)g.cs * 3u + skew;
        g.ph = (int)(colb & 3u);
        g.col4 = colb & ~3u;
        g.nd = (g.ph + 3 * g.nc + 15) >> 4;
        g.ppr = 1 + ((g.ph + 3 * (g.nc + 2) + 8 + 15) >> 4);
        return g;
    };
    // Starts the transfer of the window of destination rows [r0, r1) into the LDS slice and returns its first (virtual)
    // source row; sets nrows. A piece is 16 bytes at a dword-aligned address; the margin piece and the pieces behind the row's
    // data repeat a neighbouring data piece (their content is never read before a replica is written over it).
    int nrows = 0;
    auto issue = [&](const DmaTile &g, int r0, int r1) {
        const int a_v = to_sgpr((int)floorf(src_coord_d(pcy + r0, ry, offy, fylo)));
        const int b_v = to_sgpr((int)floorf(src_coord_d(pcy + r1 - 1, ry, offy, fylo))) + 1;
        nrows = b_v - a_v + 1;
        // every 16-byte piece of every row lies inside the batch buffer (the last rows of the last sample may not)
        const uint32_t last_row = (uint32_t)max(min(b_v, yhi), ylo) * row_stride + g.col4;
        const bool safe = (uint64_t)last_row + 16ull * (uint64_t)g.nd <= (uint64_t)lim;
        if (safe) {
            // One load instruction per row and 64 pieces: the row's address and its LDS slot are scalar arithmetic, a lane
            // only adds its piece offset, the same for every row; consecutive lanes fill consecutive 16-byte slots.
            for (int c0 = 0; c0 < g.ppr; c0 += RMX_WAVE) {
                const int c = c0 + lane;
                const uint32_t lane_off = 16u * (uint32_t)max(min(c - 1, g.nd - 1), 0);
                if (c < g.ppr) {
                    for (int r = 0; r < nrows; r++) {
                        const int ysrc = max(min(a_v + r, yhi), ylo);
                        const uint8_t *rowp = base4 + ((uint32_t)ysrc * row_stride + g.col4);
                        if constexpr (!(RMX_DMA_EXPERIMENT & 1))
                            __builtin_amdgcn_global_load_lds((glb_ptr_t)(rowp + lane_off), (lds_ptr_t)(bufb + (r * g.ppr + c0) * 16), 16, 0, RMX_LDS_LOAD_AUX);
                    }
                }
            }
        } else {
            // the window touches the last bytes of the batch buffer: bounds-checked byte loads, stored by the lanes
            const int tp = nrows * g.ppr;
            for (int idx = lane; idx < tp; idx += RMX_WAVE) {
                const int r = idx / g.ppr;
                const int c = idx - r * g.ppr;
                const int ysrc = max(min(a_v + r, yhi), ylo);
                const int piece = max(min(c - 1, g.nd - 1), 0);
                const uint32_t off = (uint32_t)ysrc * row_stride + g.col4 + 16u * (uint32_t)piece;
                uint32_t w[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint32_t v = 0;
#pragma unroll
                    for (int b = 0; b < 4; b++) {
                        const uint32_t ob = off + 4u * i + b;
                        v |= (ob < lim ? (uint32_t)base4[ob] : 0u) << (8 * b);
                    }
                    w[i] = v;
                }
                lds_u32 *dst4 = (lds_u32 *)(bufb + 16 * idx);
                dst4[0] = w[0]; dst4[1] = w[1]; dst4[2] = w[2]; dst4[3] = w[3];
            }
        }
        return a_v;
    };
    // A lane's x taps in a tile: byte offset of the left neighbour inside an LDS row (dword part and byte phase), weights
    uint32_t bo4[PX], bsh[PX];
    float wx[PX], omx[PX];
    int G = 1, lr = 0, x0 = 0, cnt = PX;
    bool lane_on = false;
    auto taps = [&](const DmaTile &g) {
        const int L = ALIGNED ? g.tw / PX : (g.tw + PX - 1) / PX;  // lanes per destination row
        G = RMX_WAVE / L;                                          // destination rows per pass
        lr = lane / L;
        int t0 = g.xt + (lane - lr * L) * PX;
        const int last = g.xt + g.tw - 1;  // last column of the tile
        if constexpr (!ALIGNED) {
            // The short last group of a row moves left until it is whole: it then recomputes up to seven pixels of the group
            // before it and stores the same values to the same places, and every lane has 8 pixels, 16-byte stores and no
            // element-wise path (which, taken by one lane, costs the wavefront half a pass more). Only a tile narrower than 8
            // pixels keeps a short group.
            if (g.tw >= PX) t0 = min(t0, last + 1 - PX);
            cnt = min(PX, last + 1 - t0);
        }
        lane_on = lr < G && cnt > 0;
#pragma unroll
        for (int k = 0; k < PX; k++) {
            // (pixels behind a partial group repeat the tile's last column: their taps stay inside the window, they are not stored)
            const int col = ALIGNED ? t0 + k : min(t0 + k, last);
            const float sx = src_coord_d(pcx + col, rx, offx, fxlo);
            const float fx = floorf(sx);
            wx[k] = sx - fx;
            omx[k] = 1.0f - wx[k];
            const uint32_t b = (uint32_t)(16 + g.ph + 3 * ((int)fx - g.cs));
            bo4[k] = b & ~3u;
            bsh[k] = b & 3u;
        }
        x0 = hf ? (dw - t0 - cnt) : t0;
    };

    // The wavefront's windows, tile by tile and top to bottom inside a tile. The stores of a window's last pass are held back
    // in registers until the next window's loads have been started (the LDS slice is free once the blend has read it):
    // memory operations of a wavefront complete in issue order, so the wait for those loads, which allows the DEFERRED
    // youngest operations (the held-back stores) to be outstanding, never waits for a store to reach memory.
    constexpr bool DEFER = sizeof(T) <= 2;  // (an fp32 run is 24 registers: stored at once)
    // The FEWEST store instructions a held-back group can become (more are harmless, fewer would let a load slip through the
    // wait): three planes are three instructions; an interleaved run is contiguous and the compiler merges its stores up to
    // 16 bytes each: 48 bytes of fp16 are three, 24 bytes of u8 two. tests/test_dma_waitcnt_cpu.py checks the generated code.
    constexpr int DEFERRED = (LAYOUT == RMX_NHWC && sizeof(T) == 1) ? 2 : 3;
    int tile = 0, r0 = r_begin;
    DmaTile g = tile_geom(0);
    int a_v = issue(g, r0, min(r0 + wrows, r_end));
    taps(g);  // while the loads are in flight
    bool held = false;
    for (;;) {
        const int r1 = min(r0 + wrows, r_end);
        // The compiler does not order LDS reads behind the loads into LDS: await them explicitly, between two fences.
        if (DEFER && held) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(DEFERRED) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wave_sync();
        const int pitch_b = g.ppr * 16;
        // clamp-to-edge: the pixel before the window's first column repeats it, the two after its last column repeat that
        if (g.rep_l || g.rep_r) {
            for (int rr = lane; rr < nrows; rr += RMX_WAVE) {
                lds_u8 *row = bufb + rr * pitch_b + 16 + g.ph;
                if (g.rep_l) {
#pragma unroll
                    for (int b = 0; b < 3; b++) row[b - 3] = row[b];
                }
                if (g.rep_r) {
                    lds_u8 *lastpx = row + 3 * (g.nc - 1);
#pragma unroll
                    for (int b = 0; b < 3; b++) lastpx[3 + b] = lastpx[6 + b] = lastpx[b];
                }
            }
            wave_sync();
        }

        // ---- blend, epilogue, store: G rows per pass
        PackedGroup<T> packed;
        bool packed_on = false;
        int packed_r = 0;
        for (int rs = r0; rs < r1; rs += G) {
            const int r = rs + lr;
            const bool on = lane_on && r < r1;
            bool full = on;  // lanes with a whole group of 8 pixels (the any-width form stores a short last group element-wise, at once)
            if (on) {
                float sy = src_coord_d(pcy + r, ry, offy, fylo);
                float fy = floorf(sy);
                float wy = sy - fy;
                const lds_u8 *row0 = bufb + ((int)fy - a_v) * pitch_b;
                const lds_u8 *row1 = row0 + pitch_b;
                const float omy = 1.0f - wy;
                float v[3][PX];
#pragma unroll
                for (int k = 0; k < PX; k++) {
                    if constexpr (RMX_DMA_EXPERIMENT & 4) {
                        const float t = k ? v[0][0] : __builtin_bit_cast(float, *(const lds_u32 *)(row0 + bo4[0]) + *(const lds_u32 *)(row1 + bo4[0]));
                        v[0][k] = v[1][k] = v[2][k] = t;
                        continue;
                    }
                    const lds_u32 *q0 = (const lds_u32 *)(row0 + bo4[k]);
                    const lds_u32 *q1 = (const lds_u32 *)(row1 + bo4[k]);
                    const uint32_t a0 = q0[0], a1 = q0[1], a2 = q0[2], b0 = q1[0], b1 = q1[1], b2 = q1[2];
                    // tl = R G B of the left neighbour and R of the right one; tr = G B of the right one
                    const uint32_t tl = __builtin_amdgcn_alignbyte(a1, a0, bsh[k]), tr = __builtin_amdgcn_alignbyte(a2, a1, bsh[k]);
                    const uint32_t bl = __builtin_amdgcn_alignbyte(b1, b0, bsh[k]), br = __builtin_amdgcn_alignbyte(b2, b1, bsh[k]);
                    float w00 = omy * omx[k], w01 = omy * wx[k], w10 = wy * omx[k];
                    float o0 = __builtin_fmaf(ubyte0(tl), w00, __builtin_fmaf(ubyte3(tl), w01, __builtin_fmaf(ubyte0(bl), w10, ubyte3(bl) * wy * wx[k])));
                    float o1 = __builtin_fmaf(ubyte1(tl), w00, __builtin_fmaf(ubyte0(tr), w01, __builtin_fmaf(ubyte1(bl), w10, ubyte0(br) * wy * wx[k])));
                    float o2 = __builtin_fmaf(ubyte2(tl), w00, __builtin_fmaf(ubyte1(tr), w01, __builtin_fmaf(ubyte2(bl), w10, ubyte1(br) * wy * wx[k])));
                    if constexpr (QUANT) {
                        // (a convex blend of bytes stays inside 0..255: rounding is the whole u8 store rule here)
                        o0 = __builtin_rintf(o0); o1 = __builtin_rintf(o1); o2 = __builtin_rintf(o2);
                    }
                    chain_colour<CHAIN>(o0, o1, o2, cp, sh2, sh4, ctab);
                    if constexpr (NORM) {
                        o0 = __builtin_fmaf(o0, sc[0], bi[0]); o1 = __builtin_fmaf(o1, sc[1], bi[1]); o2 = __builtin_fmaf(o2, sc[2], bi[2]);
                    }
                    v[0][k] = o0; v[1][k] = o1; v[2][k] = o2;
                }
                if constexpr (!ALIGNED) full = cnt == PX;
                if (full) pack_group<T, LAYOUT>(v, hf, packed);
                else store_group<T, LAYOUT, PX, RMX_DMA_NT>(dimg, a.dst_h, a.dst_w, r, x0, cnt, v, hf);
            }
            if (DEFER && rs + G >= r1) {  // the window's last pass: held back
                packed_on = full;
                packed_r = r;
            } else if (full) {
                if constexpr (RMX_DMA_EXPERIMENT & 2) keep_alive(packed);
                else store_packed<T, LAYOUT, RMX_DMA_NT, !ALIGNED>(dimg, a.dst_h, a.dst_w, r, x0, packed);
            }
        }

        // ---- the next window: its loads first, then the held-back stores
        int nr0 = r0 + wrows, ntile = tile;
        if (nr0 >= r_end) {
            nr0 = r_begin;
            ntile = tile + 1;
        }
        const bool more = ntile < ntx;
        DmaTile ng = g;
        wave_sync();  // the blend has read the LDS slice for the last time
        if (more) {
            if (ntile != tile) ng = tile_geom(ntile);
            a_v = issue(ng, nr0, min(nr0 + wrows, r_end));
        }
        asm volatile("" ::: "memory");  // the held-back stores are issued after those loads, not before
        if (DEFER && packed_on) {
            if constexpr (RMX_DMA_EXPERIMENT & 2) keep_alive(packed);
            else store_packed<T, LAYOUT, RMX_DMA_NT, !ALIGNED>(dimg, a.dst_h, a.dst_w, packed_r, x0, packed);
        }
        asm volatile("" ::: "memory");
        if (!more) break;
        // (the aligned form always holds stores back: lane 0 has a whole group in every last pass; a tile of the any-width
        // form that is narrower than 8 pixels has none, and then no store was issued behind the loads)
        held = ALIGNED ? true : (__builtin_amdgcn_ballot_w64(packed_on) != 0);
        if (ntile != tile) taps(ng);  // while the loads are in flight
        g = ng;
        tile = ntile;
        r0 = nr0;
    }
}

template <typename T, int LAYOUT, bool ALIGNED>
static KernelFn pick3(bool norm, bool quant, int chain) {
    if (norm && quant && chain == CHAIN_LINEAR) return (KernelFn)rmx_resize_dma_kernel<T, LAYOUT, true, true, CHAIN_LINEAR, ALIGNED>;
    if (norm && quant && chain == CHAIN_TWIST) return (KernelFn)rmx_resize_dma_kernel<T, LAYOUT, true, true, CHAIN_TWIST, ALIGNED>;
    if (norm && quant) return (KernelFn)rmx_resize_dma_kernel<T, LAYOUT, true, true, CHAIN_NONE, ALIGNED>;
    if (norm) return (KernelFn)rmx_resize_dma_kernel<T, LAYOUT, true, false, CHAIN_NONE, ALIGNED>;
    return (KernelFn)rmx_resize_dma_kernel<T, LAYOUT, false, false, CHAIN_NONE, ALIGNED>;
}

// aligned: the variant for whole groups and 16-byte aligned rows; null for the one combination that variant leaves to the
// staged fast kernel (interleaved fp32). The other variant takes every format.
KernelFn select_resize_dma_kernel(int dtype, int layout, bool norm, bool quant, int chain, bool aligned, const char **name) {
    *name = "rmx_resize_dma_kernel";
    if (!aligned) {
        if (layout == RMX_NCHW) {
            switch (dtype) {
                case RMX_FP32: return pick3<float, RMX_NCHW, false>(norm, quant, chain);
                case RMX_FP16: return pick3<__half, RMX_NCHW, false>(norm, quant, chain);
                default: return pick3<uint8_t, RMX_NCHW, false>(norm, quant, chain);
            }
        }
        switch (dtype) {
            case RMX_FP32: return pick3<float, RMX_NHWC, false>(norm, quant, chain);
            case RMX_FP16: return pick3<__half, RMX_NHWC, false>(norm, quant, chain);
            default: return pick3<uint8_t, RMX_NHWC, false>(norm, quant, chain);
        }
    }
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return pick3<float, RMX_NCHW, true>(norm, quant, chain);
            case RMX_FP16: return pick3<__half, RMX_NCHW, true>(norm, quant, chain);
            default: return pick3<uint8_t, RMX_NCHW, true>(norm, quant, chain);
        }
    }
    switch (dtype) {
        case RMX_FP32: return nullptr;
        case RMX_FP16: return pick3<__half, RMX_NHWC, true>(norm, quant, chain);
        default: return pick3<uint8_t, RMX_NHWC, true>(norm, quant, chain);
    }
}

}  // namespace rmx
