// K2t streaming path: triangular (antialiased) downscaling for batches in which every source row starts at the same byte
// phase (row stride a multiple of 4). Same arithmetic as rmx_resize_tri_down_kernel (rmx_kernels_tri.hip), operation for
// operation: a wavefront owns 128 output columns (two per lane) and a strip of output rows, filters its source rows
// horizontally in ascending order and adds each filtered row, from registers, to the output rows in flight (four slots).
// What differs is how the source rows reach the horizontal pass:
//   * rows travel from global memory straight into LDS (global_load_lds_dwordx4: 16 bytes per lane, no vector register, no
//     unpacking, no LDS store instruction). An LDS row holds the raw packed-RGB bytes: a margin for the left edge replicas,
//     then the row's bytes from the dword that holds the tile's first source pixel, then room for the right replicas. The
//     row's address and LDS slot are scalar arithmetic; a lane adds its 16-byte piece offset, a constant of the tile;
//   * a ring of four row slots: while two rows are filtered, the loads of the next two are in flight;
//   * a column's taps are 3 x taps consecutive bytes at any byte phase: read as aligned dwords, realigned with v_alignbyte
//     (one per 4 bytes), then unpacked byte by byte as before.
// The kernel spends its time issuing instructions (vector, scalar and LDS alike: four wavefronts per SIMD cannot hide one
// another's issue slots), and this form needs about 40 % fewer per source row than staging through registers (per lane and
// row: 16-byte loads, realignment to one dword per pixel, LDS stores and their addresses).
#pragma once
#include "rmx_device.h"
#include "rmx_launch.h"
#include "rmx_tri_math.h"

#include <type_traits>

// Wavefronts per SIMD the register budget is set for (a workgroup of 256 threads is one wavefront per SIMD): 96 registers,
// met without spills. Measured on 1080p -> 640 x 360: a budget for six gains nothing, for four loses a fifth. (Also measured:
// touching the rows of the step after next ahead of the loads, to have them in L2: 65.8 against 60.6 us.)
#ifndef RMX_TDMA_WAVES
#define RMX_TDMA_WAVES 5
#endif

namespace rmx {

extern __shared__ uint32_t rmx_lds_tdma[];

typedef __attribute__((address_space(3))) float lds_f32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// the coefficients of one source row for the SLOTS output rows in flight, as one LDS access
template <int SLOTS> struct SlotVec;
template <> struct SlotVec<4> { typedef f32x4 type; };
template <> struct SlotVec<2> { typedef f32x2 type; };
typedef float f32x8 __attribute__((ext_vector_type(8)));
template <> struct SlotVec<8> { typedef f32x8 type; };

constexpr int TS_RPS = 2;    // source rows per step; the ring holds two steps
constexpr int TS_NCH = 2;    // load instructions per row at most (64 pieces of 16 bytes each)
constexpr int TS_TAB = 64;   // source rows of the table of vertical coefficients
constexpr int TS_EDGE = 16;  // passes of an edge row at most (= vertical taps the host admits)

template <int B>
RMX_DEV float ubyte_at(uint32_t v) {
    if constexpr (B == 0) return ubyte0(v);
    else if constexpr (B == 1) return ubyte1(v);
    else if constexpr (B == 2) return ubyte2(v);
    else return ubyte3(v);
}

// One tap of the horizontal pass: pixel PIX of the realigned dwords e[] (3 bytes from byte 3 PIX), three FMAs.
template <int PIX, int NE>
RMX_DEV void tri_tap(const uint32_t (&e)[NE], float c, float &a0, float &a1, float &a2) {
    constexpr int B = 3 * PIX;
    a0 = __builtin_fmaf(ubyte_at<B & 3>(e[B >> 2]), c, a0);
    a1 = __builtin_fmaf(ubyte_at<(B + 1) & 3>(e[(B + 1) >> 2]), c, a1);
    a2 = __builtin_fmaf(ubyte_at<(B + 2) & 3>(e[(B + 2) >> 2]), c, a2);
}

// NT taps of one column, the first at pixel OFF of e[]
template <int NT, int NE, int OFF = 0, int K = 0>
RMX_DEV void tri_taps(const uint32_t (&e)[NE], const float (&c)[8], float &a0, float &a1, float &a2) {
    if constexpr (K < NT) {
        tri_tap<K + OFF, NE>(e, c[K], a0, a1, a2);
        tri_taps<NT, NE, OFF, K + 1>(e, c, a0, a1, a2);
    }
}

// One output element per lane as exactly one vector memory instruction (the wait for the loads into LDS counts the store
// instructions issued behind them, so their number must not be left to the compiler): `bits` to row + voff + OFF bytes.
template <typename T, int OFF>
RMX_DEV void store_elem(const T *row, uint32_t voff, uint32_t bits) {
    if constexpr (sizeof(T) == 4) asm volatile("global_store_dword %0, %1, %2 offset:%3" ::"v"(voff), "v"(bits), "s"(row), "n"(OFF) : "memory");
    else if constexpr (sizeof(T) == 2) asm volatile("global_store_short %0, %1, %2 offset:%3" ::"v"(voff), "v"(bits), "s"(row), "n"(OFF) : "memory");
    else asm volatile("global_store_byte %0, %1, %2 offset:%3" ::"v"(voff), "v"(bits), "s"(row), "n"(OFF) : "memory");
}

// acc += h * c and acc = 0 on the accumulator's own register. (Written as plain expressions, the accumulators of the rows
// in flight are renamed at every join of the row loop's paths and copied back: two dozen moves per source row.)
RMX_DEV void fmac_inplace(float &acc, float h, float c) { asm("v_fmac_f32 %0, %1, %2" : "+v"(acc) : "v"(h), "v"(c)); }
RMX_DEV void zero_inplace(float &acc) { asm("v_mov_b32 %0, 0" : "+v"(acc)); }

template <typename T>
RMX_DEV uint32_t elem_bits(float v) {
    const T o = OutCvt<T>::cvt(v);
    if constexpr (sizeof(T) == 4) return __builtin_bit_cast(uint32_t, o);
    else if constexpr (sizeof(T) == 2) return (uint32_t)__builtin_bit_cast(uint16_t, o);
    else return (uint32_t)o;
}

// SLOTS: output rows in flight. Four cover every downscale (rows four apart never share a source row); eight cover samples
// that grow vertically by up to about 3.8 (two taps, several output rows per source row; 113 registers, four wavefronts per
// SIMD), so that a batch of RandomResizedCrop windows, some of which shrink and some of which grow, stays in this kernel
// (measured on 256 such windows to 224 x 224: 160 us through the ring kernel; in that kernel a sample that shrinks runs a row
// loop of its own that adds to the lower four sets only, and windows with two or three horizontal taps have their own
// unrolled passes: 70.2 -> 67.2 us on those windows). Two are enough when
// rows two apart never do, which the host establishes for ratios that are whole or half numbers (1080 -> 360 rows, any
// decimation by 2, 3, 4 or 1.5): every source row then enters two accumulator sets instead of four.
template <typename T, int LAYOUT, bool NORM, bool QUANT, int SLOTS>
__global__ void __launch_bounds__(256, SLOTS == 8 ? 4 : RMX_TDMA_WAVES) rmx_resize_tri_dma_kernel(RmxKArgs a) {
    constexpr int TS_SLOTS = SLOTS;
    typedef typename SlotVec<SLOTS>::type slotv;
    typedef __attribute__((address_space(3))) slotv lds_slotv;
    constexpr int TPX = 2;               // columns per lane: lane and lane + 64
    constexpr int TTW = RMX_WAVE * TPX;  // output columns per wave tile
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, a.nblocks) * (uint32_t)a.wpb + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, part;
    wave_to_sample(a, wave, s, part);
    const int tiles_x = a.aux1;
    const int strip = part / tiles_x, tx = part - strip * tiles_x;
    // the whole table row in one round trip
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.pc_x), "s"(P.flags), "s"(P.rx), "s"(P.scale[0]), "s"(P.bias[2]), "s"(P.fsx));
    s = P.plan[2];  // (the host may have put the rows in another order: the row names its sample)

    const int dw = P.dst_w, dh = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows, xt = tx * TTW;
    if (r0 >= dh || xt >= dw) return;
    const int r1 = min(r0 + srows, dh);
    const int tw = min(TTW, dw - xt);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;
    const int xlo = P.src_x, ylo = P.src_y;
    const int xhi = xlo + P.src_w - 1, yhi = ylo + P.src_h - 1;
    const int pcx = P.pc_x, pcy = P.pc_y;
    const TriAxis ax = tri_axis(P.rx, P.fsx), ay = tri_axis(P.ry, P.fsy);
    const int kx = to_sgpr(ax.ksize), ky = to_sgpr(ay.ksize);
    // Accumulator sets this sample uses: output row r lives in set (r - r0) & smask. A sample that shrinks vertically never has
    // more than four rows in flight (the host has established that for every sample with a vertical ratio of 1 and more), so
    // in the kernel with eight sets it leaves the upper four alone: half the vertical FMAs per source row.
    const int smask = SLOTS == 8 ? to_sgpr(P.ry >= 1.0f ? 3 : 7) : SLOTS - 1;

    // (a sample is smaller than 4 GiB: the host checks it, so offsets inside a sample are 32-bit)
    uint32_t row_stride_v;
    const uint8_t *simg_v = sample_base(a, s, row_stride_v);
    const uint32_t row_stride = (uint32_t)to_sgpr((int)row_stride_v);
    const uint8_t *simg = reinterpret_cast<const uint8_t *>(((uint64_t)(uint32_t)to_sgpr((int)((uintptr_t)simg_v >> 32)) << 32) |
                                                            (uint32_t)to_sgpr((int)(uint32_t)(uintptr_t)simg_v));
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint8_t *base4 = simg - skew;  // dword-aligned base below the sample
    const uint64_t left = (uint64_t)((a.src + a.src_bytes) - base4);
    const uint32_t lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;  // bytes of the batch buffer from base4 on
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    // (the wavefront's index inside its workgroup comes from a lane id: wave-uniform, but only a scalar register says so)
    const uint32_t slice_off = (uint32_t)to_sgpr((int)((uint32_t)wib * (uint32_t)a.lds_bytes));
    lds_u8 *bufb = (lds_u8 *)(lds_ptr_t)rmx_lds_tdma + slice_off;

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    // ---- the tile's source columns and the layout of an LDS row (all wave-uniform)
    int l_first, l_last;
    {
        int lf, ll;
        float w0;
        tri_loc(ax, pcx + xt, (float)xlo, lf, w0);
        tri_loc(ax, pcx + xt + tw - 1, (float)xlo, ll, w0);
        l_first = to_sgpr(lf);
        l_last = to_sgpr(ll);
    }
    const int cs = max(min(l_first, xhi), xlo);
    const int ce = max(min(l_last + kx - 1, xhi), xlo);
    const int nrep_l = max(cs - l_first, 0), nrep_r = max(l_last + kx - 1 - ce, 0);
    const uint32_t colb = (uint32_t)cs * 3u + skew;
    const int ph = (int)(colb & 3u);        // byte phase of pixel cs inside its dword
    const uint32_t col4 = colb & ~3u;       // byte offset (from base4) of that dword, within a row
    const int nd = (ph + 3 * (ce - cs + 1) + 15) >> 4;  // data pieces of a row
    const int lm = ((3 * nrep_l + 15) >> 4) << 4;        // margin bytes in front of the data
    // data, right replicas, and the bytes the widest tap read (8 taps from the last column's first tap) may touch
    const int body = max(ph + 3 * (l_last + 8 - cs) + 8, 16 * nd);
    const int pitch = lm + (((body + 15) >> 4) << 4);
    const int ppr = pitch >> 4;  // pieces per row
    const int tab_off = a.lds_bytes - (SLOTS > 4 ? SLOTS : 4) * (TS_TAB + TS_EDGE) * 4;  // the tables of vertical coefficients (sized for four slots at least)
    // (the host sizes the slice for four rows of the widest tile; a tile that does not fit is left alone)
    if (2 * TS_RPS * pitch > tab_off || ppr > TS_NCH * RMX_WAVE || 3 * (nrep_l + nrep_r) > RMX_WAVE) return;

    // ---- output rows of the strip, one per lane (a strip has at most 64 rows): first tap row and its weight offset;
    // wave-uniform code fetches a row's entry with v_readlane
    int oloc_v;
    float ow0_v;
    tri_loc(ay, pcy + min(r0 + lane, r1 - 1), (float)ylo, oloc_v, ow0_v);
    auto row_loc = [&](int r) { return __builtin_amdgcn_readlane(oloc_v, r - r0); };
    auto row_w0 = [&](int r) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ow0_v), r - r0)); };
    auto last_tap_row = [&](int r) { return max(min(row_loc(r) + ky - 1, yhi), ylo); };
    const int y_first = max(min(row_loc(r0), yhi), ylo);
    const int y_last = last_tap_row(r1 - 1);

    // ---- load plan of the tile: piece c of an LDS row is loaded by lane c & 63 of load instruction c >> 6. Margin pieces
    // and pieces behind the data repeat a neighbouring data piece (their content is never read before a replica is written
    // over it), so no load leaves the row's own bytes.
    uint32_t lane_off[TS_NCH];
    bool piece_on[TS_NCH];
#pragma unroll
    for (int k = 0; k < TS_NCH; k++) {
        const int c = k * RMX_WAVE + lane;
        lane_off[k] = 16u * (uint32_t)max(min(c - (lm >> 4), nd - 1), 0);
        piece_on[k] = c < ppr;
    }
    // Rows from y_lanes on are stored by the lanes, with bounds-checked loads: those whose last piece would leave the batch
    // buffer, which only the last row of the last sample of the buffer can be (a row's pieces end less than 16 bytes behind
    // the row); should even the row before it not fit, every row goes that way.
    const uint32_t tail = col4 + 16u * (uint32_t)nd;
    int y_lanes = y_last + 1;
    if ((uint64_t)((uint32_t)y_last * row_stride) + tail > (uint64_t)lim)
        y_lanes = (y_last > y_first && (uint64_t)((uint32_t)(y_last - 1) * row_stride) + tail <= (uint64_t)lim) ? y_last : y_first;

    // Starts the transfer of the next two source rows (rows behind the last repeat it) into the two slots of one half of the
    // ring; y_next / roff_next walk down the rows. Returns whether a row was stored by the lanes.
    int y_next = y_first;
    uint32_t roff_next = (uint32_t)y_first * row_stride + col4;
    auto issue = [&](lds_u8 *half_base) {
        bool by_lanes = false;
#pragma unroll
        for (int q = 0; q < TS_RPS; q++) {
            const uint32_t roff = roff_next;
            lds_u8 *slot = half_base + q * pitch;
            if (y_next < y_lanes) {
                const uint8_t *rowp = base4 + roff;
#pragma unroll
                for (int k = 0; k < TS_NCH; k++) {
                    if (k * RMX_WAVE < ppr) {
                        if (piece_on[k]) __builtin_amdgcn_global_load_lds((glb_ptr_t)(rowp + lane_off[k]), (lds_ptr_t)(slot + k * RMX_WAVE * 16), 16, 0, RMX_LDS_LOAD_AUX);
                    }
                }
            } else {
                by_lanes = true;
                for (int c = lane; c < ppr; c += RMX_WAVE) {
                    const uint32_t off = roff + 16u * (uint32_t)max(min(c - (lm >> 4), nd - 1), 0);
                    lds_u32 *dst4 = (lds_u32 *)(slot + 16 * c);
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
            if (y_next < y_last) {
                y_next++;
                roff_next += row_stride;
            }
        }
        return by_lanes;
    };

    // The first two rows are asked for here, ahead of the coefficient set-up below (some hundred instructions that need no
    // memory): they travel while it runs.
    const bool first_by_lanes = issue(bufb);

    // ---- per-lane columns: taps, coefficients (registers), column sums, destination column (mirrored if asked)
    // (a lane whose column lies beyond the row takes the last column again and stores the same value to the same place:
    // every store instruction is then issued by every wavefront, which the count in the wait below relies on)
    // Neighbouring columns per lane (2 l and 2 l + 1 instead of l and l + 64) when the horizontal ratio is 2 or 3 exactly: the
    // first taps of neighbouring columns then lie exactly 2 or 3 source pixels apart with the same coefficients (every product
    // and sum of the coordinate law is exact), their tap ranges overlap, and one read of the union serves both: for ratio 3
    // (five taps after the first, whose coefficient is 0) 8 pixels instead of 2 x 5, i.e. 24 byte -> float conversions
    // instead of 30 and 7 LDS dwords instead of 10 per source row. pair_r is the ratio, or 0: columns 64 apart. Established on
    // the tile's first two columns with the law itself; even tile widths only (a lane beyond the row takes the last pair again).
    int pair_r = 0;
    if constexpr (SLOTS != 8) {
        const int R = (int)P.rx;
        if ((R == 2 || R == 3) && P.rx == (float)R && !(tw & 1) && kx == 2 * R) {
            int l0, l1;
            float wa, wb;
            tri_loc(ax, pcx + xt, (float)xlo, l0, wa);
            tri_loc(ax, pcx + xt + 1, (float)xlo, l1, wb);
            const bool first_is_zero = tri_coeff(wa, ax.radius, 0, ax.fscale) == 0.0f;
            if (l1 == l0 + R && wa == wb && first_is_zero == (R == 3)) pair_r = R;
        }
        pair_r = to_sgpr(pair_r);
    }
    const int pair_lane = min(lane, (tw >> 1) - 1);
    uint32_t xoff[TPX], tap_w[TPX], tap_ph[TPX];
    float colsum[TPX], creg[TPX][8];
    int locx[TPX];
    float w0x[TPX];
    bool lead = false;  // some column's first tap has a coefficient other than 0
#pragma unroll
    for (int i = 0; i < TPX; i++) {
        const int col = pair_r ? xt + 2 * pair_lane + i : xt + lane + RMX_WAVE * i;
        const int colc = min(col, dw - 1);
        xoff[i] = (uint32_t)(hf ? (dw - 1 - colc) : colc) * (uint32_t)(LAYOUT == RMX_NCHW ? sizeof(T) : 3 * sizeof(T));
        tri_loc(ax, pcx + colc, (float)xlo, locx[i], w0x[i]);
        float sum = 0.0f;
        for (int k = 0; k < kx; k++) sum += tri_coeff(w0x[i], ax.radius, k, ax.fscale);
        colsum[i] = (sum == 0.0f) ? 1.0f : sum;
        lead = lead || !(tri_coeff(w0x[i], ax.radius, 0, ax.fscale) == 0.0f);
    }
    // When the first tap of every column of the tile has coefficient 0 (ratios 1 and 3, the odd whole numbers: the first tap then
    // lies a whole radius from the centre), the horizontal pass starts one pixel on with one tap less: fma(p, 0, 0) is the 0
    // the accumulation starts from anyway. Wave-uniform.
    const int skip = (kx > 1 && __builtin_amdgcn_ballot_w64(lead) == 0) ? 1 : 0;
    const int kx_run = kx - skip;
#pragma unroll
    for (int i = 0; i < TPX; i++) {
#pragma unroll
        for (int k = 0; k < 8; k++) creg[i][k] = (k < kx_run) ? tri_coeff(w0x[i], ax.radius, k + skip, ax.fscale) : 0.0f;
        // the first tap's byte inside an LDS row (a tap left of the window reads a replica in or behind the margin)
        const uint32_t tb = (uint32_t)(lm + ph + 3 * (locx[i] + skip - cs));
        tap_w[i] = tb & ~3u;
        tap_ph[i] = tb & 3u;
    }
    // sum of the vertical coefficients of output row r0 + lane, taps ascending; the row that completes fetches its sum from
    // the lane that holds it
    float rsum_v = 0.0f;
    for (int j = 0; j < ky; j++) rsum_v += tri_coeff(ow0_v, ay.radius, j, ay.fscale);
    rsum_v = (rsum_v == 0.0f) ? 1.0f : rsum_v;

    // ---- clamp-to-edge columns: byte e of the replicas (left ones first) is copied by lane e from the first / last pixel
    const int nrep_b = 3 * (nrep_l + nrep_r);
    uint32_t rep_src, rep_dst;
    {
        const int e = lane;
        const bool is_l = e < 3 * nrep_l;
        const int er = is_l ? e : e - 3 * nrep_l;
        const int j = er / 3, c = er - 3 * j;
        rep_src = (uint32_t)(lm + ph + (is_l ? 0 : 3 * (ce - cs)) + c);
        rep_dst = (uint32_t)(lm + ph + (is_l ? -3 * (j + 1) : 3 * (ce - cs + 1 + j)) + c);
    }
    auto replicate = [&](lds_u8 *half_base, int nr) {
        if (nrep_b > 0) {
            if (lane < nrep_b) {
                for (int q = 0; q < nr; q++) {
                    lds_u8 *slot = half_base + q * pitch;
                    slot[rep_dst] = slot[rep_src];
                }
            }
            wave_sync();
        }
    };

    // ---- output rows in flight: row r accumulates in slot (r - r0) & 3 until its last tap row has been added. rq is the
    // oldest row in flight, qlast its last tap row (wave-uniform state).
    float acc[TS_SLOTS][3][TPX];
#pragma unroll
    for (int m = 0; m < TS_SLOTS; m++)
#pragma unroll
        for (int c = 0; c < 3; c++)
#pragma unroll
            for (int i = 0; i < TPX; i++) acc[m][c][i] = 0.0f;
    int rq = r0;
    int qlast = last_tap_row(r0);
    int emitted = 0;  // output rows stored since the loads of the rows in work were started

    // ---- vertical coefficients by source row, a table of 64 rows x 4 slots in the tail of the LDS slice: entry (l, k) is
    // the coefficient with which source row ytab + l enters the output row of slot k (0: none; fma(h, 0, acc) == acc for
    // the finite h a filtered row is, so all four slots take every row and no branch is needed). Lane l writes row l; the
    // filter loop reads a row's entry with one broadcast read. Rebuilt every 64 source rows. The first and the last row
    // of the window serve several taps of a row each (clamped tap indices) and take their own path below.
    lds_f32 *cftab = (lds_f32 *)(bufb + tab_off);
    const lds_slotv *cv_next = (const lds_slotv *)cftab;  // the table entry of the next source row
    int ytab = y_first;
    auto build_table = [&]() {
        const int y = ytab + lane;
        float cf[TS_SLOTS];
#pragma unroll
        for (int k = 0; k < TS_SLOTS; k++) cf[k] = 0.0f;
        for (int rb = r0; rb < r1; rb += smask + 1) {
#pragma unroll
            for (int k = 0; k < TS_SLOTS; k++) {
                const int r = rb + k;
                if (k <= smask && r < r1) {
                    const int j = y - row_loc(r);
                    const float c = tri_coeff(row_w0(r), ay.radius, j, ay.fscale);
                    if ((uint32_t)j < (uint32_t)ky) cf[k] = c;
                }
            }
        }
        slotv cfv;
#pragma unroll
        for (int k = 0; k < TS_SLOTS; k++) cfv[k] = cf[k];
        *(lds_slotv *)(cftab + TS_SLOTS * lane) = cfv;
        wave_sync();
    };

    // An output row whose last tap row has been added: normalise, epilogue, store; its slot starts again at zero. orow walks
    // down the output rows (planar: the row of channel 0; the other planes lie `plane` elements on).
    T *orow = dimg + (size_t)r0 * a.dst_w * (LAYOUT == RMX_NCHW ? 1 : 3);
    const size_t plane = (size_t)a.dst_h * a.dst_w;
    const int orow_step = a.dst_w * (LAYOUT == RMX_NCHW ? 1 : 3);
    int rsum_idx = 0;
    // 1 / (row sum x column sum) is kept from one output row to the next: rows of an integer ratio all have the same sum,
    // and the division is a dozen instructions per column
    int rsum_bits_prev = 0;  // (no row sum is +0: a zero sum is replaced by 1)
    float inv_c[TPX];
#pragma unroll
    for (int i = 0; i < TPX; i++) inv_c[i] = 0.0f;
    auto emit = [&](auto slot) {
        constexpr int M = decltype(slot)::value;
        const int rsum_bits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, rsum_v), rsum_idx);
        if (rsum_bits != rsum_bits_prev) {
            rsum_bits_prev = rsum_bits;
            const float rsum = __builtin_bit_cast(float, rsum_bits);
#pragma unroll
            for (int i = 0; i < TPX; i++) inv_c[i] = 1 / (rsum * colsum[i]);
        }
#pragma unroll
        for (int i = 0; i < TPX; i++) {
            const float inv = inv_c[i];
#pragma unroll
            for (int ch = 0; ch < 3; ch++) {
                float t = acc[M][ch][i] * inv;
                zero_inplace(acc[M][ch][i]);
                if constexpr (QUANT) t = round_u8(t);
                if constexpr (NORM) t = __builtin_fmaf(t, sc[ch], bi[ch]);
                // wave-uniform row pointer + the lane's column offset
                if constexpr (LAYOUT == RMX_NCHW) store_elem<T, 0>(orow + ch * plane, xoff[i], elem_bits<T>(t));
                else if (ch == 0) store_elem<T, 0>(orow, xoff[i], elem_bits<T>(t));
                else if (ch == 1) store_elem<T, (int)sizeof(T)>(orow, xoff[i], elem_bits<T>(t));
                else store_elem<T, 2 * (int)sizeof(T)>(orow, xoff[i], elem_bits<T>(t));
            }
        }
    };

    // The row in ring slot `slot` is source row yy: filter it and add it to the output rows in flight. NT = taps of the
    // unrolled horizontal pass (4, 5, 6 or 8 >= the taps that are run): taps beyond those carry coefficient 0 (fma(p, 0, a) == a
    // for the finite p an unpacked byte always is), so no bound test is needed inside. A column's 3 NT bytes start at byte
    // tap_ph of dword tap_w: NE + 1 dwords are read and realigned into NE.
    auto process_row = [&](auto nt, auto lower_only, auto pair, const lds_u8 *srow, int yy) {
        constexpr int NT = decltype(nt)::value;
        constexpr int PR = decltype(pair)::value;  // the lane's two columns are neighbours whose first taps lie PR pixels apart; 0: not
        // LIVE: the accumulator sets this instance of the row loop adds to and stores from (the lower four of eight for a sample
        // that shrinks: a loop of its own rather than a branch around the upper sets' FMAs, at whose join the accumulators
        // would be copied)
        constexpr int LIVE = (TS_SLOTS == 8 && decltype(lower_only)::value) ? 4 : TS_SLOTS;
        constexpr int NE = (3 * NT + 3) / 4;
        // A row inside the window is one tap of every output row that reads it: one pass, coefficients from the table. The
        // first / last row of the window is also read by every tap index that leaves the window: one pass per such tap, in
        // tap order, coefficients computed here by lane p for pass p (rare: twice per image column of strips at most).
        const lds_slotv *cvp = cv_next++;
        int npass = 1;
        if ((uint32_t)(yy - ylo - 1) >= (uint32_t)(yhi - ylo - 1)) {  // yy == ylo or yy == yhi (rows lie inside the window)
            float ec[TS_SLOTS];
            npass = 0;
#pragma unroll
            for (int m = 0; m < TS_SLOTS; m++) {
                const int r = rq + ((m - (rq - r0)) & smask);  // the row in flight that lives in slot m
                ec[m] = 0.0f;
                if (m <= smask && r < r1) {
                    const int loc = row_loc(r);
                    const int jlo = max((yy == ylo) ? 0 : yy - loc, 0);
                    const int jhi = min((yy == yhi) ? ky - 1 : yy - loc, ky - 1);
                    npass = max(npass, jhi - jlo + 1);
                    const int j = jlo + lane;
                    const float c = tri_coeff(row_w0(r), ay.radius, j, ay.fscale);
                    if (j <= jhi) ec[m] = c;
                }
            }
            lds_f32 *etab = cftab + TS_SLOTS * TS_TAB;
            slotv ecv;
#pragma unroll
            for (int m = 0; m < TS_SLOTS; m++) ecv[m] = ec[m];
            if (lane < TS_EDGE) *(lds_slotv *)(etab + TS_SLOTS * lane) = ecv;
            wave_sync();
            cvp = (const lds_slotv *)etab;
            npass = max(npass, 1);
        }
        slotv cv4 = cvp[0];
        float h[3][TPX];
        if constexpr (PR > 0) {
            // one read of the union of both columns' taps: NT + PR pixels from the first column's first tap
            constexpr int NEP = (3 * (NT + PR) + 3) / 4;
            uint32_t w[NEP + 1];
            const lds_u32 *p0 = (const lds_u32 *)(srow + tap_w[0]);
#pragma unroll
            for (int j = 0; j <= NEP; j++) w[j] = p0[j];
            uint32_t e[NEP];
#pragma unroll
            for (int j = 0; j < NEP; j++) e[j] = __builtin_amdgcn_alignbyte(w[j + 1], w[j], tap_ph[0]);
            float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, b0 = 0.0f, b1 = 0.0f, b2 = 0.0f;
            tri_taps<NT, NEP, 0>(e, creg[0], a0, a1, a2);
            tri_taps<NT, NEP, PR>(e, creg[1], b0, b1, b2);
            h[0][0] = a0; h[1][0] = a1; h[2][0] = a2;
            h[0][1] = b0; h[1][1] = b1; h[2][1] = b2;
        } else {
            uint32_t w[TPX][NE + 1];
#pragma unroll
            for (int i = 0; i < TPX; i++) {
                const lds_u32 *p0 = (const lds_u32 *)(srow + tap_w[i]);
#pragma unroll
                for (int j = 0; j <= NE; j++) w[i][j] = p0[j];
            }
#pragma unroll
            for (int i = 0; i < TPX; i++) {
                uint32_t e[NE];
#pragma unroll
                for (int j = 0; j < NE; j++) e[j] = __builtin_amdgcn_alignbyte(w[i][j + 1], w[i][j], tap_ph[i]);
                float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f;
                tri_taps<NT, NE>(e, creg[i], a0, a1, a2);
                h[0][i] = a0;
                h[1][i] = a1;
                h[2][i] = a2;
            }
        }
        // ---- vertical pass: every pass adds the filtered row to all four slots with that pass's coefficients (0: none)
        for (int p = 0;;) {
#pragma unroll
            for (int m = 0; m < LIVE; m++)
#pragma unroll
                for (int ch = 0; ch < 3; ch++)
#pragma unroll
                    for (int i = 0; i < TPX; i++) fmac_inplace(acc[m][ch][i], h[ch][i], cv4[m]);
            if (++p >= npass) break;
            cv4 = cvp[p];
        }
        // ---- rows whose last tap was this source row
        while (qlast <= yy) {
            if constexpr (TS_SLOTS == 2) {
                if (rsum_idx & 1) emit(std::integral_constant<int, 1>{});
                else emit(std::integral_constant<int, 0>{});
            } else if constexpr (LIVE == 8) {
                switch (rsum_idx & 7) {
                    case 0: emit(std::integral_constant<int, 0>{}); break;
                    case 1: emit(std::integral_constant<int, 1>{}); break;
                    case 2: emit(std::integral_constant<int, 2>{}); break;
                    case 3: emit(std::integral_constant<int, 3>{}); break;
                    case 4: emit(std::integral_constant<int, 4>{}); break;
                    case 5: emit(std::integral_constant<int, 5>{}); break;
                    case 6: emit(std::integral_constant<int, 6>{}); break;
                    default: emit(std::integral_constant<int, 7>{}); break;
                }
            } else {
                switch (rsum_idx & 3) {
                    case 0: emit(std::integral_constant<int, 0>{}); break;
                    case 1: emit(std::integral_constant<int, 1>{}); break;
                    case 2: emit(std::integral_constant<int, 2>{}); break;
                    default: emit(std::integral_constant<int, 3>{}); break;
                }
            }
            rq++;
            rsum_idx++;
            orow += orow_step;
            emitted++;
            qlast = rq < r1 ? last_tap_row(rq) : 0x7fffffff;  // (behind the last row: no source row completes anything)
        }
    };

    // Two rows per step. The loads of a step were started a step earlier; the compiler does not order LDS reads behind
    // loads into LDS, so their arrival is awaited explicitly, between two wavefront fences. Memory operations of a wavefront
    // complete in issue order, loads and stores on one counter: the wait names the number of store instructions issued
    // since those loads (6 per output row, see store_elem), so it never waits for a store. The next step's loads are
    // started right behind the wait (the slots they fill were read for the last time in the step before).
    constexpr int NS = 3 * TPX;  // store instructions per output row
    auto run = [&](auto nt, auto lower_only, auto pair) {
        lds_u8 *half_cur = bufb, *half_nxt = bufb + TS_RPS * pitch;
        bool by_lanes = first_by_lanes;
        build_table();  // (under the round trip of the first loads)
        for (int y = y_first; y <= y_last; y += TS_RPS) {
            const int nr = min(TS_RPS, y_last - y + 1);
            if (y + nr - ytab > RMX_WAVE) {
                ytab = y;
                cv_next = (const lds_slotv *)cftab;
                build_table();
            }
            if (by_lanes || emitted > 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // (the lanes' own loads, or many rows)
            else if (emitted == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else if (emitted == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NS) : "memory");
            else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NS) : "memory");
            wave_sync();
            emitted = 0;
            by_lanes = (y + TS_RPS <= y_last) ? issue(half_nxt) : false;
            replicate(half_cur, nr);
            for (int q = 0; q < nr; q++) process_row(nt, lower_only, pair, half_cur + q * pitch, y + q);
            wave_sync();  // the slots are reused two steps on
            lds_u8 *t = half_cur;
            half_cur = half_nxt;
            half_nxt = t;
        }
    };
    // (two and three taps: windows that grow or barely shrink horizontally, which only batches with growing samples hold in numbers)
    auto run_taps = [&](auto lower_only) {
        constexpr std::integral_constant<int, 0> apart{};
        if constexpr (SLOTS != 8) {
            if (pair_r == 2 && kx_run == 4) {
                run(std::integral_constant<int, 4>{}, lower_only, std::integral_constant<int, 2>{});
                return;
            }
            if (pair_r == 3 && kx_run == 5) {
                run(std::integral_constant<int, 5>{}, lower_only, std::integral_constant<int, 3>{});
                return;
            }
        }
        if (SLOTS == 8 && kx_run <= 2) run(std::integral_constant<int, SLOTS == 8 ? 2 : 4>{}, lower_only, apart);
        else if (SLOTS == 8 && kx_run == 3) run(std::integral_constant<int, SLOTS == 8 ? 3 : 4>{}, lower_only, apart);
        else if (kx_run <= 4) run(std::integral_constant<int, 4>{}, lower_only, apart);
        else if (kx_run == 5) run(std::integral_constant<int, 5>{}, lower_only, apart);
        else if (kx_run <= 6) run(std::integral_constant<int, 6>{}, lower_only, apart);
        else run(std::integral_constant<int, 8>{}, lower_only, apart);
    };
    if (SLOTS == 8 && smask == 3) run_taps(std::integral_constant<bool, SLOTS == 8>{});
    else run_taps(std::false_type{});
}

template <typename T, int LAYOUT, int SLOTS>
static KernelFn pick3_tdma(bool norm, bool quant) {
    if (norm && quant) return (KernelFn)rmx_resize_tri_dma_kernel<T, LAYOUT, true, true, SLOTS>;
    if (norm) return (KernelFn)rmx_resize_tri_dma_kernel<T, LAYOUT, true, false, SLOTS>;
    return (KernelFn)rmx_resize_tri_dma_kernel<T, LAYOUT, false, false, SLOTS>;
}

// The instances of one (accumulator sets, layout) pair, one translation unit each so that they compile side by side
// (rmx_kernels_tri_dma*.hip); rmx_kernels_tri_dma.hip picks among them.
#define RMX_TDMA_UNIT(SLOTS, LAYOUT, NAME)                                    \
    KernelFn NAME(int dtype, bool norm, bool quant) {                         \
        switch (dtype) {                                                      \
            case RMX_FP32: return pick3_tdma<float, LAYOUT, SLOTS>(norm, quant);   \
            case RMX_FP16: return pick3_tdma<__half, LAYOUT, SLOTS>(norm, quant);  \
            default: return pick3_tdma<uint8_t, LAYOUT, SLOTS>(norm, quant);  \
        }                                                                     \
    }

KernelFn tdma_unit_2_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_2_nhwc(int dtype, bool norm, bool quant);
KernelFn tdma_unit_4_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_4_nhwc(int dtype, bool norm, bool quant);
KernelFn tdma_unit_8_nchw(int dtype, bool norm, bool quant);
KernelFn tdma_unit_8_nhwc(int dtype, bool norm, bool quant);

}  // namespace rmx
