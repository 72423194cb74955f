// K2t: triangular (antialiased) resize, separable, both passes staged through LDS, with the
// same epilogue as the bilinear kernel ([u8 quantise] -> [mirror] -> [normalise] -> layout -> cast).
//
// A wavefront owns an x-tile of 128 output columns (two per lane) and a strip of output rows
// and walks down the strip with a ring of horizontally filtered source rows in its private LDS
// slice:
//   horizontal pass  one source row at a time: stage the row segment (dword per pixel), then
//                    every lane accumulates its two columns over the kx taps in tap order
//                    (coefficients come from a per-tile LDS table built once per strip);
//   vertical pass    per output row: accumulate the ky ring rows in tap order, normalise by
//                    1/(rowsum*colsum), epilogue, store.
// Source rows enter the ring exactly once per strip; the intermediate never touches HBM.
#include "rmx_device.h"
#include "rmx_launch.h"
#include "rmx_tri_math.h"

#include <type_traits>

// Wavefronts per SIMD the register budget of the downscaling kernel is set for, by columns per lane (a workgroup of 256
// threads is one wavefront per SIMD): 128 registers with two columns, 96 with one.
#ifndef RMX_TRI_DOWN_WAVES
#define RMX_TRI_DOWN_WAVES(npx) ((npx) == 1 ? 5 : 4)
#endif

namespace rmx {

extern __shared__ uint32_t rmx_lds_tri[];

constexpr int TTW = 128;  // output columns per wave tile
constexpr int TPX = 2;    // columns per lane
constexpr int TRB = 3;    // source rows staged per batch (one memory round trip per batch, not per row)

template <typename T, int LAYOUT, bool NORM, bool QUANT>
__global__ void __launch_bounds__(256) rmx_resize_tri_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, gridDim.x) * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, part;
    wave_to_sample(a, wave, s, part);
    const int tiles_x = a.aux1;
    const int strip = part / tiles_x, tx = part - strip * tiles_x;
    const RmxSample &P = a.table[s];
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
    const int kx = ax.ksize, ky = ay.ksize;
    const int ring_rows = P.strip_rows >> 16;      // power of two
    const int kx_cap = P.strip_rows & 0xffff;
    const int ring_mask = ring_rows - 1;

    uint32_t row_stride32;
    const uint8_t *simg = sample_base(a, s, row_stride32);
    const size_t row_stride = row_stride32;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    // LDS slice: coef[kx_cap][TTW] | ring[ring_rows][3][TTW] | srcrow[TRB][...]
    uint32_t *base = rmx_lds_tri + (size_t)wib * (a.lds_bytes >> 2);
    // (the coefficient table exists only for kernels of more than 8 taps; shorter ones keep them in registers)
    float *coef = reinterpret_cast<float *>(base);
    float *ring = coef + (kx_cap > 8 ? kx_cap * TTW : 0);
    uint32_t *srcrow = reinterpret_cast<uint32_t *>(ring + ring_rows * 3 * TTW);

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    // ---- per-lane column taps (two columns), coefficient table, column sums
    const int t0 = xt + lane * TPX;
    const int cnt = max(0, min(TPX, dw - t0));
    int locx[TPX];
    float colsum[TPX];
#pragma unroll
    for (int i = 0; i < TPX; i++) {
        int u = pcx + min(t0 + i, dw - 1);
        float w0;
        tri_loc(ax, u, (float)xlo, locx[i], w0);
        float sum = 0.0f;
        for (int k = 0; k < kx; k++) {
            float c = tri_coeff(w0, ax.radius, k, ax.fscale);
            if (kx_cap > 8) coef[k * TTW + lane * TPX + i] = c;
            sum += c;
        }
        colsum[i] = (sum == 0.0f) ? 1.0f : sum;
    }
    // register copies of the coefficients for the short-kernel path of the horizontal pass
    const bool short_taps = kx_cap <= 8;  // kx <= kx_cap
    float creg[TPX][8];
#pragma unroll
    for (int i = 0; i < TPX; i++) {
        int u = pcx + min(t0 + i, dw - 1);
        float w0;
        int loc;
        tri_loc(ax, u, (float)xlo, loc, w0);
#pragma unroll
        for (int k = 0; k < 8; k++) creg[i][k] = (k < kx) ? tri_coeff(w0, ax.radius, k, ax.fscale) : 0.0f;
    }
    // tile-wide staged source column range (wave-uniform)
    int l_first, l_last;
    {
        float w0;
        tri_loc(ax, pcx + xt, (float)xlo, l_first, w0);
        tri_loc(ax, pcx + xt + tw - 1, (float)xlo, l_last, w0);
    }
    const int cs = max(min(l_first, xhi), xlo);
    const int ce = max(min(l_last + kx - 1, xhi), xlo);
    const int items = (ce - cs + 4) >> 2;
    // staged row: [lpad: copies of the first column][items*4 pixels from column cs][copies of the last column].
    // With the border columns repeated in LDS no tap index needs clamping in the horizontal pass.
    const int nrep_l = max(cs - l_first, 0), nrep_r = max(l_last + kx - 1 - ce, 0);
    const int lpad = (nrep_l + 3) & ~3;
    const int spitch = lpad + items * 4 + ((nrep_r + 3) & ~3);  // dwords per staged row
    wave_sync();

    int next_row;
    {
        int loc;
        float w0;
        tri_loc(ay, pcy + r0, (float)ylo, loc, w0);
        next_row = max(min(loc, yhi), ylo);
    }

    for (int r = r0; r < r1; r++) {
        int locy;
        float w0y;
        tri_loc(ay, pcy + r, (float)ylo, locy, w0y);
        const int rb = max(min(locy + ky - 1, yhi), ylo);
        // ---- horizontal pass for the source rows that enter the window
        while (next_row <= rb) {
            // stage up to TRB rows with one round trip: (row, item) pairs form one flat index space, four
            // loads per lane are issued back to back before the first is consumed
            const int nb = min(TRB, rb - next_row + 1);
            const int total = nb * items;
            const float inv_items = 1.0f / (float)items;
            for (int base = 0; base < total; base += 4 * RMX_WAVE) {
                uint32_t w[4][3];
                int dsto[4];
                const uint8_t *pp[4];
                bool safe = true;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int idx = min(base + i * RMX_WAVE + lane, total - 1);
                    const int q = (int)(((float)idx + 0.5f) * inv_items);  // idx / items (exact: see the bilinear kernel)
                    const int j = idx - q * items;
                    pp[i] = simg + ((uint32_t)__mul24(next_row + q, (int)row_stride) + (uint32_t)(cs + 4 * j) * 3u);
                    dsto[i] = q * spitch + lpad + 4 * j;
                    safe = safe && (pp[i] - ((uintptr_t)pp[i] & 3u) + 16 <= buf_end);
                }
                if (safe) {
                    u32x4_a4 t[4];
                    uint32_t ph[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        ph[i] = (uint32_t)((uintptr_t)pp[i] & 3u);
                        t[i] = *reinterpret_cast<const u32x4_a4 *>(pp[i] - ph[i]);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        w[i][0] = __builtin_amdgcn_alignbyte(t[i].y, t[i].x, ph[i]);
                        w[i][1] = __builtin_amdgcn_alignbyte(t[i].z, t[i].y, ph[i]);
                        w[i][2] = __builtin_amdgcn_alignbyte(t[i].w, t[i].z, ph[i]);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) load_realigned<4>(pp[i], buf_end, w[i]);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    uint4 px;
                    px.x = w[i][0];
                    px.y = __builtin_amdgcn_alignbyte(w[i][1], w[i][0], 3);
                    px.z = __builtin_amdgcn_alignbyte(w[i][2], w[i][1], 2);
                    px.w = w[i][2] >> 8;
                    if (base + i * RMX_WAVE + lane < total) *reinterpret_cast<uint4 *>(srcrow + dsto[i]) = px;
                }
            }
            wave_sync();
            if (nrep_l + nrep_r > 0) {
                const int per_row = nrep_l + nrep_r;
                for (int e = lane; e < nb * per_row; e += RMX_WAVE) {
                    const int q = e / per_row, z = e - q * per_row;
                    uint32_t *srow = srcrow + q * spitch + lpad;
                    if (z < nrep_l) srow[-1 - z] = srow[0];
                    else srow[(ce - cs) + 1 + (z - nrep_l)] = srow[ce - cs];
                }
                wave_sync();
            }
            for (int q = 0; q < nb; q++) {
                const uint32_t *srow = srcrow + q * spitch + lpad;
                float *slot = ring + ((next_row + q) & ring_mask) * 3 * TTW;
#pragma unroll
                for (int i = 0; i < TPX; i++) {
                    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f;
                    if (short_taps) {
                        // up to 8 taps: fixed offsets from one address, coefficients from registers, unrolled
                        // for 4, 6 or 8 taps. Taps beyond kx carry coefficient 0 (fma(p, 0, a) == a for the
                        // finite p an unpacked byte always is), so no bound test is needed inside.
                        const uint32_t *p0 = srow + (locx[i] - cs);
                        auto run = [&](auto nt) {
#pragma unroll
                            for (int k = 0; k < decltype(nt)::value; k++) {
                                const uint32_t p = p0[k];
                                a0 = __builtin_fmaf(ubyte0(p), creg[i][k], a0);
                                a1 = __builtin_fmaf(ubyte1(p), creg[i][k], a1);
                                a2 = __builtin_fmaf(ubyte2(p), creg[i][k], a2);
                            }
                        };
                        if (kx <= 4) run(std::integral_constant<int, 4>{});
                        else if (kx <= 6) run(std::integral_constant<int, 6>{});
                        else run(std::integral_constant<int, 8>{});
                    } else {
                        for (int k = 0; k < kx; k++) {
                            const uint32_t p = srow[locx[i] + k - cs];
                            const float c = coef[k * TTW + lane * TPX + i];
                            a0 = __builtin_fmaf(ubyte0(p), c, a0);
                            a1 = __builtin_fmaf(ubyte1(p), c, a1);
                            a2 = __builtin_fmaf(ubyte2(p), c, a2);
                        }
                    }
                    slot[0 * TTW + lane * TPX + i] = a0;
                    slot[1 * TTW + lane * TPX + i] = a1;
                    slot[2 * TTW + lane * TPX + i] = a2;
                }
            }
            wave_sync();
            next_row += nb;
        }
        // ---- vertical pass (each lane reads only ring entries it wrote itself)
        if (cnt > 0) {
            float rsum = 0.0f;
            for (int j = 0; j < ky; j++) rsum += tri_coeff(w0y, ay.radius, j, ay.fscale);
            rsum = (rsum == 0.0f) ? 1.0f : rsum;
            float acc[3][TPX];
#pragma unroll
            for (int c = 0; c < 3; c++)
#pragma unroll
                for (int i = 0; i < TPX; i++) acc[c][i] = 0.0f;
            // taps in ascending order; coefficient and ring row are found once per tap for both columns
            for (int j = 0; j < ky; j++) {
                const int rr = max(min(locy + j, yhi), ylo);
                const float *slot = ring + (rr & ring_mask) * 3 * TTW + lane * TPX;
                const float c = tri_coeff(w0y, ay.radius, j, ay.fscale);
#pragma unroll
                for (int i = 0; i < TPX; i++) {
                    acc[0][i] = __builtin_fmaf(slot[0 * TTW + i], c, acc[0][i]);
                    acc[1][i] = __builtin_fmaf(slot[1 * TTW + i], c, acc[1][i]);
                    acc[2][i] = __builtin_fmaf(slot[2 * TTW + i], c, acc[2][i]);
                }
            }
            float v[3][TPX];
#pragma unroll
            for (int i = 0; i < TPX; i++) {
                const float inv = 1 / (rsum * colsum[i]);
                v[0][i] = acc[0][i] * inv;
                v[1][i] = acc[1][i] * inv;
                v[2][i] = acc[2][i] * inv;
            }
#pragma unroll
            for (int c = 0; c < 3; c++)
#pragma unroll
                for (int i = 0; i < TPX; i++) {
                    float t = v[c][i];
                    if constexpr (QUANT) t = round_u8(t);
                    if constexpr (NORM) t = __builtin_fmaf(t, sc[c], bi[c]);
                    v[c][i] = t;
                }
            const int x0 = hf ? (dw - t0 - cnt) : t0;
            store_group<T, LAYOUT, TPX>(dimg, a.dst_h, a.dst_w, r, x0, cnt, v, hf);
        }
    }
}

// Downscaling variant (vertical ratio >= 1, at most 8 horizontal taps): the vertical pass keeps no ring of
// filtered rows. Source rows are filtered horizontally in ascending order and each filtered row is added,
// straight from registers, to the output rows whose windows contain it; at a ratio >= 1 a source row belongs
// to the windows of at most four consecutive output rows (the host checks this per sample), so four sets of
// accumulators in a shift register are enough. Every output row still receives its taps in ascending order
// with the same coefficients, so the result is bit-identical to the ring kernel's, and the LDS slice shrinks
// to the staged source rows of one round of loads. A lane owns columns lane and lane + 64 of the tile:
// neighbouring lanes read source pixels `ratio` dwords apart, half the bank stride of adjacent column pairs.
constexpr int TDM = 4;  // output rows in flight

template <typename T, int LAYOUT, bool NORM, bool QUANT, int NPX>
__global__ void __launch_bounds__(256, RMX_TRI_DOWN_WAVES(NPX)) rmx_resize_tri_down_kernel(RmxKArgs a) {
    constexpr int TPX = NPX;            // columns per lane: lane, lane + 64, ...
    constexpr int TTW = RMX_WAVE * NPX;  // output columns per wave tile
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
    const int kx = ax.ksize, ky = ay.ksize;

    // (a sample is smaller than 4 GiB: the host checks it, so offsets inside a sample are 32-bit)
    uint32_t row_stride;
    const uint8_t *simg = sample_base(a, s, row_stride);
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint8_t *base4 = simg - skew;  // dword-aligned base below the sample
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *srcrow = rmx_lds_tri + (size_t)wib * (a.lds_bytes >> 2);

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    // tile-wide staged source column range (wave-uniform)
    int l_first, l_last;
    {
        float w0;
        tri_loc(ax, pcx + xt, (float)xlo, l_first, w0);
        tri_loc(ax, pcx + xt + tw - 1, (float)xlo, l_last, w0);
    }
    const int cs = max(min(l_first, xhi), xlo);
    const int ce = max(min(l_last + kx - 1, xhi), xlo);
    const int items = (ce - cs + 4) >> 2;
    // staged row: [lpad: copies of the first column][items*4 pixels from column cs][copies of the last column].
    // With the border columns repeated in LDS no tap index needs clamping in the horizontal pass.
    const int nrep_l = max(cs - l_first, 0), nrep_r = max(l_last + kx - 1 - ce, 0);
    const int lpad = (nrep_l + 3) & ~3;
    const int spitch = lpad + items * 4 + ((nrep_r + 3) & ~3);  // dwords per staged row

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

    // ---- staging plan of the tile. A row is `items` four-pixel items; a round is four 16-byte loads per lane:
    // 4 rows of one slot, 2 rows of two slots or 1 row of up to four slots (a row has at most 3 x 64 items at up
    // to 8 taps; spare slots repeat the last one). Everything that does not depend on the row is computed here:
    // the dword-aligned byte offset of the slot's item inside a row, the byte phase (the same for all items of a
    // lane, they are 12 bytes apart) and the item's place in the staged row.
    const int spr = (items + RMX_WAVE - 1) / RMX_WAVE;
    const int sh = spr == 1 ? 0 : (spr == 2 ? 1 : 2);  // log2(slots per row)
    // every wide load of this wavefront stays inside the batch buffer (last row, last item, carry and load width)
    // (rows longer than the three slots of a round take the row-by-row path as well)
    const bool safe = items <= 3 * RMX_WAVE && simg + ((size_t)y_last * row_stride + (size_t)(cs + 4 * (items - 1)) * 3 + 3 + 4 + 16) <= buf_end;
    // rows per round, never more than the slice holds (then the spare slots repeat a row); the bounds-checked path
    // stages one row at a time. (The tail of the slice holds the table of vertical coefficients.)
    const int rpr = safe ? min(4 >> sh, max(1, ((a.lds_bytes >> 2) - TDM * RMX_WAVE) / spitch)) : 1;
    // (the item's byte offset in memory follows from its place in the staged row: 3 bytes per dword, which is recomputed per
    // load rather than kept in four more registers)
    uint32_t sl_lds[4];
    bool sl_on[4];
    const uint32_t low = ((uint32_t)cs * 3u) & 3u;  // (items are 12 bytes apart: one phase for the whole row)
    const uint32_t al_base = (((uint32_t)cs * 3u) & ~3u) - 3u * (uint32_t)lpad;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int k = min(i & ((1 << sh) - 1), spr - 1);
        const int j = min(lane + RMX_WAVE * k, items - 1);
        sl_lds[i] = (uint32_t)(lpad + 4 * j);
        sl_on[i] = lane + RMX_WAVE * k < items;
    }

    // A round of loads. (Issuing the first round here, ahead of the set-up of the coefficients below, was measured: the 16
    // registers it keeps busy make the compiler spill inside the filter loop, 86 us instead of 73.)
    u32x4_a4 t[4];
    auto issue = [&](int yb, int nr) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int q = min(i >> sh, nr - 1);
            const uint32_t ro = (uint32_t)(yb + q) * row_stride + skew;  // wave-uniform: row start from base4
            const uint32_t r = ro & 3u;
            uint32_t place = sl_lds[i];
            asm volatile("" : "+v"(place));  // (keeps the product below inside the loop)
            t[i] = *reinterpret_cast<const u32x4_a4 *>(base4 + (((ro - r) + al_base + ((low + r) & 4u)) + 3u * place));
        }
    };
    // ---- per-lane columns: taps, coefficients (registers), column sums, destination column (mirrored if asked)
    int locx[TPX];
    bool col_on[TPX];
    uint32_t xcol[TPX];
    float colsum[TPX], creg[TPX][8];
#pragma unroll
    for (int i = 0; i < TPX; i++) {
        const int col = xt + lane + RMX_WAVE * i;
        col_on[i] = col < dw;
        const int colc = min(col, dw - 1);
        xcol[i] = (uint32_t)(hf ? (dw - 1 - colc) : colc);
        float w0;
        tri_loc(ax, pcx + colc, (float)xlo, locx[i], w0);
        float sum = 0.0f;
        for (int k = 0; k < kx; k++) sum += tri_coeff(w0, ax.radius, k, ax.fscale);
        colsum[i] = (sum == 0.0f) ? 1.0f : sum;
#pragma unroll
        for (int k = 0; k < 8; k++) creg[i][k] = (k < kx) ? tri_coeff(w0, ax.radius, k, ax.fscale) : 0.0f;
    }
    // byte offsets of a lane's first taps inside a staged row
    uint32_t tap_ofs[TPX];
#pragma unroll
    for (int i = 0; i < TPX; i++) tap_ofs[i] = (uint32_t)(lpad + locx[i] - cs) * 4u;

    // sum of the vertical coefficients of output row r0 + lane, taps ascending; the row that completes fetches its sum from
    // the lane that holds it
    float rsum_v = 0.0f;
    for (int j = 0; j < ky; j++) rsum_v += tri_coeff(ow0_v, ay.radius, j, ay.fscale);
    rsum_v = (rsum_v == 0.0f) ? 1.0f : rsum_v;

    // ---- output rows in flight: row r accumulates in slot (r - r0) & 3 until its last tap row has been added. rq is the
    // oldest row in flight, qlast its last tap row (wave-uniform state).
    float acc[TDM][3][TPX];
#pragma unroll
    for (int m = 0; m < TDM; m++)
#pragma unroll
        for (int c = 0; c < 3; c++)
#pragma unroll
            for (int i = 0; i < TPX; i++) acc[m][c][i] = 0.0f;
    int rq = r0;
    int qlast = last_tap_row(r0);

    // ---- vertical coefficients by source row, a table of 64 rows x 4 slots in the tail of the LDS slice: entry (l, k) is
    // the coefficient with which source row ytab + l enters the output row of slot k (0: none; fma(h, 0, acc) == acc for
    // the finite h a filtered row is, so all four slots take every row and no branch is needed). Lane l writes row l; the
    // filter loop reads a row's entry with one broadcast read. Rebuilt every 64 source rows. The first and the last row
    // of the window serve several taps of a row each (clamped tap indices) and take their own path below.
    float *cftab = reinterpret_cast<float *>(srcrow + ((a.lds_bytes >> 2) - TDM * RMX_WAVE));
    int ytab = y_first;
    auto build_table = [&]() {
        const int y = ytab + lane;
        float cf[TDM];
#pragma unroll
        for (int k = 0; k < TDM; k++) cf[k] = 0.0f;
        for (int rb = r0; rb < r1; rb += TDM) {
#pragma unroll
            for (int k = 0; k < TDM; k++) {
                const int r = rb + k;
                if (r < r1) {
                    const int j = y - row_loc(r);
                    const float c = tri_coeff(row_w0(r), ay.radius, j, ay.fscale);
                    if ((uint32_t)j < (uint32_t)ky) cf[k] = c;
                }
            }
        }
        *reinterpret_cast<float4 *>(cftab + TDM * lane) = make_float4(cf[0], cf[1], cf[2], cf[3]);
        wave_sync();
    };
    // clamp-to-edge columns of the nr staged rows
    auto replicate = [&](int nr) {
        if (nrep_l + nrep_r > 0) {
            const int per_row = nrep_l + nrep_r;
            for (int e = lane; e < nr * per_row; e += RMX_WAVE) {
                const int q = e / per_row, z = e - q * per_row;
                uint32_t *srow = srcrow + q * spitch + lpad;
                if (z < nrep_l) srow[-1 - z] = srow[0];
                else srow[(ce - cs) + 1 + (z - nrep_l)] = srow[ce - cs];
            }
            wave_sync();
        }
    };

    // An output row whose last tap row has been added: normalise, epilogue, store; its slot starts again at zero.
    auto emit = [&](auto slot) {
        constexpr int M = decltype(slot)::value;
        const float rsum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, rsum_v), rq - r0));
#pragma unroll
        for (int i = 0; i < TPX; i++) {
            const float inv = 1 / (rsum * colsum[i]);
#pragma unroll
            for (int ch = 0; ch < 3; ch++) {
                float t = acc[M][ch][i] * inv;
                acc[M][ch][i] = 0.0f;
                if constexpr (QUANT) t = round_u8(t);
                if constexpr (NORM) t = __builtin_fmaf(t, sc[ch], bi[ch]);
                // wave-uniform row pointer + the lane's column offset
                if constexpr (LAYOUT == RMX_NCHW) {
                    T *rowp = dimg + ((size_t)ch * a.dst_h + rq) * a.dst_w;
                    if (col_on[i]) rowp[xcol[i]] = OutCvt<T>::cvt(t);
                } else {
                    T *rowp = dimg + (size_t)rq * a.dst_w * 3 + ch;
                    if (col_on[i]) rowp[xcol[i] * 3u] = OutCvt<T>::cvt(t);
                }
            }
        }
    };

    // staged row q is source row yy: filter it and add it to the output rows in flight. NT = taps of the unrolled
    // horizontal pass (4, 6 or 8 >= kx): taps beyond kx carry coefficient 0 (fma(p, 0, a) == a for the finite p
    // an unpacked byte always is), so no bound test is needed inside; all LDS reads go out before the arithmetic.
    auto process_row = [&](auto nt, int q, int yy) {
        constexpr int NT = decltype(nt)::value;
        const uint8_t *srow = reinterpret_cast<const uint8_t *>(srcrow) + (uint32_t)(q * spitch) * 4u;
        uint32_t px[TPX][NT];
        const float4 cv4 = *reinterpret_cast<const float4 *>(cftab + TDM * (yy - ytab));
#pragma unroll
        for (int i = 0; i < TPX; i++) {
            const uint32_t *p0 = reinterpret_cast<const uint32_t *>(srow + tap_ofs[i]);
#pragma unroll
            for (int k = 0; k < NT; k++) px[i][k] = p0[k];
        }
        float h[3][TPX];
#pragma unroll
        for (int i = 0; i < TPX; i++) {
            float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f;
#pragma unroll
            for (int k = 0; k < NT; k++) {
                a0 = __builtin_fmaf(ubyte0(px[i][k]), creg[i][k], a0);
                a1 = __builtin_fmaf(ubyte1(px[i][k]), creg[i][k], a1);
                a2 = __builtin_fmaf(ubyte2(px[i][k]), creg[i][k], a2);
            }
            h[0][i] = a0;
            h[1][i] = a1;
            h[2][i] = a2;
        }
        // ---- vertical pass
        if (yy != ylo && yy != yhi) {
            // a row inside the window is one tap of every output row that reads it
            const float cv[TDM] = {cv4.x, cv4.y, cv4.z, cv4.w};
#pragma unroll
            for (int m = 0; m < TDM; m++)
#pragma unroll
                for (int ch = 0; ch < 3; ch++)
#pragma unroll
                    for (int i = 0; i < TPX; i++) acc[m][ch][i] = __builtin_fmaf(h[ch][i], cv[m], acc[m][ch][i]);
        } else {
            // the first / last row of the window: every tap index that leaves the window reads it too, in tap order
#pragma unroll
            for (int m = 0; m < TDM; m++) {
                const int r = rq + ((m - (rq - r0)) & (TDM - 1));  // the row in flight that lives in slot m
                if (r < r1) {
                    const int loc = row_loc(r);
                    const float w0 = row_w0(r);
                    int jlo = (yy == ylo) ? 0 : yy - loc;
                    int jhi = (yy == yhi) ? ky - 1 : yy - loc;
                    jlo = max(jlo, 0);
                    jhi = min(jhi, ky - 1);
                    for (int j = jlo; j <= jhi; j++) {
                        const float c = tri_coeff(w0, ay.radius, j, ay.fscale);
#pragma unroll
                        for (int ch = 0; ch < 3; ch++)
#pragma unroll
                            for (int i = 0; i < TPX; i++) acc[m][ch][i] = __builtin_fmaf(h[ch][i], c, acc[m][ch][i]);
                    }
                }
            }
        }
        // ---- rows whose last tap was this source row
        while (qlast <= yy && rq < r1) {
            switch ((rq - r0) & (TDM - 1)) {
                case 0: emit(std::integral_constant<int, 0>{}); break;
                case 1: emit(std::integral_constant<int, 1>{}); break;
                case 2: emit(std::integral_constant<int, 2>{}); break;
                default: emit(std::integral_constant<int, 3>{}); break;
            }
            rq++;
            qlast = last_tap_row(min(rq, r1 - 1));
        }
    };

    auto run = [&](auto nt) {
        // Software pipeline over the rounds: the loads of the next round are issued before the rows of the current
        // one are filtered and wait in registers, so a round trip to memory runs under the arithmetic of the
        // previous round. The four loads are straight-line and unconditional (rows beyond the last repeat it).
        if (safe) issue(y_first, min(rpr, y_last - y_first + 1));
        build_table();  // (under the round trip of the first loads)
        for (int y = y_first; y <= y_last;) {
            const int nr = min(rpr, y_last - y + 1);
            if (y + nr - ytab > RMX_WAVE) {
                ytab = y;
                build_table();
            }
            if (safe) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int q = min(i >> sh, nr - 1);
                    const uint32_t r = ((uint32_t)(y + q) * row_stride + skew) & 3u;
                    const uint32_t d[4] = {t[i].x, t[i].y, t[i].z, t[i].w};
                    const uint4 px = expand4(d, (low + r) & 3u);
                    if (sl_on[i]) *reinterpret_cast<uint4 *>(srcrow + (uint32_t)(q * spitch) + sl_lds[i]) = px;
                }
                wave_sync();
                const int yn = y + nr;
                issue(min(yn, y_last), max(1, min(rpr, y_last - yn + 1)));
            } else {
                // the wavefront's rows touch the last bytes of the batch buffer: row by row, bounds-checked loads
                for (int j = lane; j < items; j += RMX_WAVE) {
                    const uint8_t *pp = simg + (size_t)y * row_stride + (size_t)(cs + 4 * j) * 3;
                    uint32_t w[3];
                    load_realigned<4>(pp, buf_end, w);
                    uint4 px;
                    px.x = w[0];
                    px.y = __builtin_amdgcn_alignbyte(w[1], w[0], 3);
                    px.z = __builtin_amdgcn_alignbyte(w[2], w[1], 2);
                    px.w = w[2] >> 8;
                    *reinterpret_cast<uint4 *>(srcrow + lpad + 4 * j) = px;
                }
                wave_sync();
            }
            replicate(nr);
            for (int q = 0; q < nr; q++) process_row(nt, q, y + q);
            wave_sync();  // the next round overwrites the staged rows
            y += nr;
        }
    };
    if (kx <= 4) run(std::integral_constant<int, 4>{});
    else if (kx <= 6) run(std::integral_constant<int, 6>{});
    else run(std::integral_constant<int, 8>{});
}

template <typename T, int LAYOUT>
static KernelFn pick3(bool norm, bool quant) {
    if (norm && quant) return (KernelFn)rmx_resize_tri_kernel<T, LAYOUT, true, true>;
    if (norm) return (KernelFn)rmx_resize_tri_kernel<T, LAYOUT, true, false>;
    return (KernelFn)rmx_resize_tri_kernel<T, LAYOUT, false, false>;
}

KernelFn select_resize_tri_kernel(int dtype, int layout, bool norm, bool quant, const char **name) {
    *name = "rmx_resize_tri_kernel";
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return pick3<float, RMX_NCHW>(norm, quant);
            case RMX_FP16: return pick3<__half, RMX_NCHW>(norm, quant);
            default: return pick3<uint8_t, RMX_NCHW>(norm, quant);
        }
    }
    switch (dtype) {
        case RMX_FP32: return pick3<float, RMX_NHWC>(norm, quant);
        case RMX_FP16: return pick3<__half, RMX_NHWC>(norm, quant);
        default: return pick3<uint8_t, RMX_NHWC>(norm, quant);
    }
}

template <typename T, int LAYOUT, int NPX>
static KernelFn pick3_down(bool norm, bool quant) {
    if (norm && quant) return (KernelFn)rmx_resize_tri_down_kernel<T, LAYOUT, true, true, NPX>;
    if (norm) return (KernelFn)rmx_resize_tri_down_kernel<T, LAYOUT, true, false, NPX>;
    return (KernelFn)rmx_resize_tri_down_kernel<T, LAYOUT, false, false, NPX>;
}

template <int NPX>
static KernelFn pick_down(int dtype, int layout, bool norm, bool quant) {
    if (layout == RMX_NCHW) {
        switch (dtype) {
            case RMX_FP32: return pick3_down<float, RMX_NCHW, NPX>(norm, quant);
            case RMX_FP16: return pick3_down<__half, RMX_NCHW, NPX>(norm, quant);
            default: return pick3_down<uint8_t, RMX_NCHW, NPX>(norm, quant);
        }
    }
    switch (dtype) {
        case RMX_FP32: return pick3_down<float, RMX_NHWC, NPX>(norm, quant);
        case RMX_FP16: return pick3_down<__half, RMX_NHWC, NPX>(norm, quant);
        default: return pick3_down<uint8_t, RMX_NHWC, NPX>(norm, quant);
    }
}

// columns_per_lane: 1 (tiles of 64 output columns) or 2 (tiles of 128)
KernelFn select_resize_tri_down_kernel(int dtype, int layout, bool norm, bool quant, int columns_per_lane, const char **name) {
    *name = "rmx_resize_tri_down_kernel";
    return columns_per_lane == 1 ? pick_down<1>(dtype, layout, norm, quant) : pick_down<2>(dtype, layout, norm, quant);
}

}  // namespace rmx
