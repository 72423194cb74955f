// K2 fast path: the bilinear resize + epilogue kernel specialised for batches in which every
// written width is a multiple of 8 and the destination rows are 16-byte aligned (the training
// shapes: 224, 256, 384, 640 ...). Same arithmetic, same ring-of-rows scheme and the same
// wavefront-granular scheduling as the general kernel; what is removed is everything that only
// ragged widths need (partial groups, per-element stores, per-item bounds tests), and the
// staging addresses are a wave-uniform base plus one precomputed lane offset, so the inner
// loops are almost pure blend arithmetic.
#include "rmx_device.h"
#include "rmx_launch.h"

namespace rmx {

extern __shared__ uint32_t rmx_lds_fast[];

RMX_DEV float src_coord_f(int u, float ratio, float off, float lo) {
    float s = (float)u * ratio;
    s = s + off;
    s = s + lo;
    return s;
}

#ifdef RMX_EXP_TRACE
#define STAMP(i) do { if (a.dbg && lane == 0 && (wave % 97u) == 0u && (i) < 32) a.dbg[(wave / 97u) * 32 + (i)] = __builtin_readcyclecounter(); } while (0)
#else
#define STAMP(i) do { } while (0)
#endif

constexpr int QB = 4;  // rows per staging batch
constexpr int CB = 2;  // 64-lane chunks per row per staging batch

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Prefetch loads are written as instructions, not as C++ loads: on gfx9 the vector-memory counter
// is shared by loads and stores that may retire out of order, so as soon as a store is pending
// the compiler turns every wait into "wait for everything" and places it right behind the loads.
// Issued this way the loads stay in flight across the blend of the current step; prefetch_wait()
// is the single wait before their first use.
RMX_DEV void prefetch_load(u32x4 &dst, const uint8_t *addr) {
    // Full 64-bit vector address: a scalar-base operand would have to be produced by
    // v_readfirstlane whenever the row index comes out of the float coordinate math, and the
    // wait states that sequence needs in front of a vector-memory instruction are not inserted
    // for instructions the compiler cannot see.
    asm volatile("global_load_dwordx4 %0, %1, off\n\ts_nop 0" : "=&v"(dst) : "v"(addr) : "memory");
}

// Stores of the pipelined loop are instructions for the same reason (a pending compiler-visible
// store would drag the waits back in). s_nop covers the VALU-write -> wide-store-data hazard.
RMX_DEV void asm_store16(void *p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    u32x4 v = {a, b, c, d};
    asm volatile("s_nop 1\n\tglobal_store_dwordx4 %0, %1, off" : : "v"(p), "v"(v) : "memory");
}
RMX_DEV void asm_store8(void *p, uint32_t a, uint32_t b) {
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 v = {a, b};
    asm volatile("s_nop 1\n\tglobal_store_dwordx2 %0, %1, off" : : "v"(p), "v"(v) : "memory");
}

template <typename T, int LAYOUT>
RMX_DEV void asm_store_packed(T *sample, int H, int W, int y, int x0, const PackedGroup<T> &g) {
    constexpr int PW = PX * (int)sizeof(T) / 4;  // dwords per channel run
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T *p = sample + ((size_t)c * H + y) * W + x0;
            if constexpr (PW % 4 == 0) {
#pragma unroll
                for (int i = 0; i < PW / 4; i++)
                    asm_store16(reinterpret_cast<uint4 *>(p) + i, g.w[c * PW + 4 * i], g.w[c * PW + 4 * i + 1], g.w[c * PW + 4 * i + 2], g.w[c * PW + 4 * i + 3]);
            } else {
#pragma unroll
                for (int i = 0; i < PW / 2; i++) asm_store8(reinterpret_cast<uint2 *>(p) + i, g.w[c * PW + 2 * i], g.w[c * PW + 2 * i + 1]);
            }
        }
    } else {
        T *p = sample + ((size_t)y * W + x0) * 3;
        constexpr int TW = PackedGroup<T>::WORDS;
        if constexpr (TW % 4 == 0) {
#pragma unroll
            for (int i = 0; i < TW / 4; i++) asm_store16(reinterpret_cast<uint4 *>(p) + i, g.w[4 * i], g.w[4 * i + 1], g.w[4 * i + 2], g.w[4 * i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < TW / 2; i++) asm_store8(reinterpret_cast<uint2 *>(p) + i, g.w[2 * i], g.w[2 * i + 1]);
        }
    }
}

RMX_DEV void prefetch_wait(u32x4 (&r)[QB * CB]) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), leave expcnt/lgkmcnt alone
    static_assert(QB * CB == 8, "register list below names eight vectors");
    asm volatile("" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}

template <typename T, int LAYOUT, bool NORM, bool QUANT>
__global__ void __launch_bounds__(256) rmx_resize_fast_kernel(RmxKArgs a) {
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const int wib = threadIdx.x / RMX_WAVE;
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, gridDim.x) * (blockDim.x / RMX_WAVE) + wib;
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    STAMP(0);
    const int s = (int)(wave / (uint32_t)a.strips);
    const int strip = (int)(wave % (uint32_t)a.strips);
    const RmxSample &P = a.table[s];

    const int dw = P.dst_w, dh = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= dh || dw <= 0) return;
    const int r1 = min(r0 + srows, dh);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;

    const int xlo = P.src_x, ylo = P.src_y;
    const int xhi = xlo + P.src_w - 1, yhi = ylo + P.src_h - 1;
    const float rx = P.rx, ry = P.ry;
    const float offx = (rx - 1.0f) * 0.5f, offy = (ry - 1.0f) * 0.5f;
    const float fxlo = (float)xlo, fylo = (float)ylo;
    const int pcx = P.pc_x, pcy = P.pc_y;
    const int R = P.strip_rows;

    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;
    uint32_t *lds = rmx_lds_fast + (size_t)wib * (a.lds_bytes >> 2);

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    const uint32_t row_stride = (uint32_t)a.src_w * 3u;
    const uint8_t *simg = a.src + (size_t)s * a.src_h * row_stride;
    const uint32_t skew = (uint32_t)((uintptr_t)simg & 3u);
    const uint8_t *base4 = simg - skew;
    const uint64_t left = (uint64_t)((a.src + a.src_bytes) - base4);
    const uint32_t lim = left > 0xffffffffull ? 0xffffffffu : (uint32_t)left;

    const int tile_w = a.aux1;
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
        const int items = (nc + 3) >> 2;
        const int ipl = (items + RMX_WAVE - 1) / RMX_WAVE;
        const int pitch = 4 + items * 4 + 4;
        const uint32_t col_off = (uint32_t)cs * 3u + skew;

        // byte offsets of the left neighbour inside an LDS row, and the x weights
        uint32_t offb[PX];
        float wx[PX];
#pragma unroll
        for (int k = 0; k < PX; k++) {
            float sx = src_coord_f(pcx + t0 + k, rx, offx, fxlo);
            float fx = floorf(sx);
            wx[k] = sx - fx;
            offb[k] = (uint32_t)(4 + ((int)fx - cs)) * 4u;
        }
        // per-lane staging offsets: global bytes and LDS bytes of item `lane` of a row
        const uint32_t vo12 = 12u * (uint32_t)lane;
        const uint32_t lo16 = 16u + 16u * (uint32_t)lane;

        auto row_off = [&](int v) -> uint32_t {
            const int ysrc = max(min(v, yhi), ylo);
            return (uint32_t)ysrc * row_stride + col_off;
        };
        // loop-invariant lane offsets of the two chunks of a staging batch (clamped to the row)
        uint32_t vo[CB];
        bool okc[CB];
#pragma unroll
        for (int cl = 0; cl < CB; cl++) {
            okc[cl] = lane + RMX_WAVE * cl < items;
            vo[cl] = 12u * (uint32_t)min(lane + RMX_WAVE * cl, items - 1);
        }

        // General staging of virtual rows [new_lo, new_lo+nnew) into ring slots slot_new.. (wrapped),
        // skipping the batch of the first QB rows x first CB chunks when `skip_first`. Used for the
        // first window of a strip and for whatever does not fit the prefetch batch of the step loop.
        auto stage_general = [&](int new_lo, int nnew, int slot_new, bool skip_first, bool guarded) {
            for (int q = 0; q < nnew; q++) {
                const uint32_t ro = row_off(new_lo + q);
                int sl = slot_new + q;
                if (sl >= R) sl -= R;
                for (int j0 = (skip_first && q < QB) ? CB * RMX_WAVE : 0; j0 < items; j0 += 2 * RMX_WAVE) {
                    // two items per lane in flight
                    const int ja = j0 + lane, jb = j0 + RMX_WAVE + lane;
                    uint32_t da[4], db[4];
                    if (!guarded) {
                        u32x4_a4 va = *reinterpret_cast<const u32x4_a4 *>(base4 + (ro & ~3u) + 12u * (uint32_t)min(ja, items - 1));
                        u32x4_a4 vb = *reinterpret_cast<const u32x4_a4 *>(base4 + (ro & ~3u) + 12u * (uint32_t)min(jb, items - 1));
                        da[0] = va.x; da[1] = va.y; da[2] = va.z; da[3] = va.w;
                        db[0] = vb.x; db[1] = vb.y; db[2] = vb.z; db[3] = vb.w;
                    } else {
                        const uint32_t oa = (ro & ~3u) + 12u * (uint32_t)min(ja, items - 1);
                        const uint32_t ob = (ro & ~3u) + 12u * (uint32_t)min(jb, items - 1);
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            da[i] = (oa + 4u * i < lim) ? *reinterpret_cast<const uint32_t *>(base4 + oa + 4u * i) : 0u;
                            db[i] = (ob + 4u * i < lim) ? *reinterpret_cast<const uint32_t *>(base4 + ob + 4u * i) : 0u;
                        }
                    }
                    const uint4 pa = expand4(da, ro & 3u), pb = expand4(db, ro & 3u);
                    if (ja < items) *reinterpret_cast<uint4 *>(lds + sl * pitch + 4 + 4 * ja) = pa;
                    if (jb < items) *reinterpret_cast<uint4 *>(lds + sl * pitch + 4 + 4 * jb) = pb;
                }
            }
        };
        auto finish_rows = [&](int nnew, int slot_new) {
            wave_sync();
            if ((rep_l || rep_r) && lane < nnew) {
                int sl = slot_new + lane;
                if (sl >= R) sl -= R;
                uint32_t *row = lds + sl * pitch;
                if (rep_l) row[3] = row[4];
                if (rep_r) row[4 + nc] = row[4 + nc - 1];
            }
            wave_sync();
        };

        // gather + blend + epilogue of output row r (this lane's 8 pixels) from the ring
        auto blend = [&](int r, int base_slot, int a_k, PackedGroup<T> &packed) {
            float sy = src_coord_f(pcy + r, ry, offy, fylo);
            float fy = floorf(sy);
            float wy = sy - fy;
            int s0 = base_slot + ((int)fy - a_k);
            if (s0 >= R) s0 -= R;
            int s1 = s0 + 1;
            if (s1 >= R) s1 -= R;
            const uint8_t *row0 = reinterpret_cast<const uint8_t *>(lds) + (uint32_t)(s0 * pitch) * 4u;
            const uint8_t *row1 = reinterpret_cast<const uint8_t *>(lds) + (uint32_t)(s1 * pitch) * 4u;
            const float omy = 1.0f - wy;
            float v[3][PX];
#pragma unroll
            for (int k = 0; k < PX; k++) {
                const uint32_t *p0 = reinterpret_cast<const uint32_t *>(row0 + offb[k]);
                const uint32_t *p1 = reinterpret_cast<const uint32_t *>(row1 + offb[k]);
                uint32_t tl = p0[0], tr = p0[1], bl = p1[0], br = p1[1];
                float omx = 1.0f - wx[k];
                float w00 = omy * omx, w01 = omy * wx[k], w10 = wy * omx;
                float o0 = __builtin_fmaf(ubyte0(tl), w00, __builtin_fmaf(ubyte0(tr), w01, __builtin_fmaf(ubyte0(bl), w10, ubyte0(br) * wy * wx[k])));
                float o1 = __builtin_fmaf(ubyte1(tl), w00, __builtin_fmaf(ubyte1(tr), w01, __builtin_fmaf(ubyte1(bl), w10, ubyte1(br) * wy * wx[k])));
                float o2 = __builtin_fmaf(ubyte2(tl), w00, __builtin_fmaf(ubyte2(tr), w01, __builtin_fmaf(ubyte2(bl), w10, ubyte2(br) * wy * wx[k])));
                // a convex blend of u8 values stays inside [0,255]: rounding alone saturates it
                if constexpr (QUANT) {
                    o0 = __builtin_rintf(o0); o1 = __builtin_rintf(o1); o2 = __builtin_rintf(o2);
                }
                if constexpr (NORM) {
                    o0 = __builtin_fmaf(o0, sc[0], bi[0]); o1 = __builtin_fmaf(o1, sc[1], bi[1]); o2 = __builtin_fmaf(o2, sc[2], bi[2]);
                }
                v[0][k] = o0; v[1][k] = o1; v[2][k] = o2;
            }
            pack_group<T, LAYOUT>(v, hf, packed);
        };

        // One prefetch batch = the first QB rows x CB chunks of a row set: all loads back to back and
        // unconditional (indices beyond the row set or the row are clamped to valid ones).
        auto issue_batch = [&](int new_lo, int nnew, u32x4 (&raw)[QB * CB], uint32_t (&ph)[QB]) {
            const uint8_t *pa[QB * CB];
#pragma unroll
            for (int ql = 0; ql < QB; ql++) {
                const uint32_t ro = row_off(new_lo + min(ql, max(nnew - 1, 0)));
                ph[ql] = ro & 3u;
#pragma unroll
                for (int cl = 0; cl < CB; cl++) pa[ql * CB + cl] = base4 + (ro & ~3u) + vo[cl];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < QB * CB; i++) {
#ifdef RMX_EXP_NOLOAD
                raw[i] = u32x4{1, 2, 3, 4};
#else
                prefetch_load(raw[i], pa[i]);
#endif
            }
        };
        auto commit_batch = [&](int nnew, int slot_new, u32x4 (&raw)[QB * CB], const uint32_t (&ph)[QB]) {
            prefetch_wait(raw);
#pragma unroll
            for (int ql = 0; ql < QB; ql++) {
                int sl = slot_new + ql;
                if (sl >= R) sl -= R;
                uint8_t *rowl = reinterpret_cast<uint8_t *>(lds + sl * pitch) + lo16;
                if (ql < nnew) {  // wave-uniform: rows beyond the set were only loaded to keep the loads unconditional
#pragma unroll
                    for (int cl = 0; cl < CB; cl++) {
                        if (cl < ipl) {
                            const uint32_t d[4] = {raw[ql * CB + cl].x, raw[ql * CB + cl].y, raw[ql * CB + cl].z, raw[ql * CB + cl].w};
                            const uint4 px = expand4(d, ph[ql]);
                            if (okc[cl]) *reinterpret_cast<uint4 *>(rowl + 1024 * cl) = px;
                        }
                    }
                }
            }
        };

        int a_k = (int)floorf(src_coord_f(pcy + r0, ry, offy, fylo));
        int b_k = (int)floorf(src_coord_f(pcy + min(r0 + G, r1) - 1, ry, offy, fylo)) + 1;
        int base_slot = 0;
        // the strip is "safe" unless its last source row reaches the end of the batch buffer
        const int b_last = (int)floorf(src_coord_f(pcy + r1 - 1, ry, offy, fylo)) + 1;
        const bool safe = ((row_off(b_last) & ~3u) + 12u * (uint32_t)items + 8u <= lim);
        // pipelined loop: usable when every later window of the strip fits one prefetch batch
        const bool pipelined = safe && ipl <= CB && (P.flags >> 16) <= (uint32_t)QB;
        if (pipelined) {
            // first window: one batch, plus (rarely) a fifth row the general way
            u32x4 raw0[QB * CB];
            uint32_t ph0[QB];
            const int n0 = b_k - a_k + 1;
            issue_batch(a_k, n0, raw0, ph0);
            commit_batch(n0, 0, raw0, ph0);
            if (n0 > QB) stage_general(a_k + QB, n0 - QB, QB, false, false);
        } else {
            stage_general(a_k, b_k - a_k + 1, 0, false, !safe);
        }
        STAMP(1);
        finish_rows(b_k - a_k + 1, 0);
        STAMP(2);
        int stamp = 3;
        (void)stamp;
        const int x0 = hf ? (dw - t0 - PX) : t0;

        if (pipelined) {
            for (int rs = r0; rs < r1; rs += G) {
                const int re = min(rs + G, r1) - 1;
                // ---- next step's window: start its loads before this step's arithmetic. QB rows x
                //      CB chunks, back to back and unconditional (indices beyond the row set or the
                //      row are clamped to valid ones).
                u32x4 raw[QB * CB];
                uint32_t ph[QB];
                const bool has_next = rs + G < r1;
                int a_n = a_k, b_n = b_k, new_lo = 0, nnew = 0, slot_new = 0, base_slot_n = base_slot;
                if (has_next) {
                    a_n = (int)floorf(src_coord_f(pcy + rs + G, ry, offy, fylo));
                    b_n = (int)floorf(src_coord_f(pcy + min(rs + 2 * G, r1) - 1, ry, offy, fylo)) + 1;
                    base_slot_n = base_slot + (a_n - a_k);
                    while (base_slot_n >= R) base_slot_n -= R;
                    new_lo = max(b_k + 1, a_n);
                    nnew = b_n - new_lo + 1;
                    slot_new = base_slot_n + (new_lo - a_n);
                    if (slot_new >= R) slot_new -= R;
                    issue_batch(new_lo, nnew, raw, ph);
                }
                STAMP(stamp); stamp++;

                const int r = rs + lr;
                const bool mine = lane_on && r <= re;
                PackedGroup<T> packed;
#ifdef RMX_EXP_NOBLEND
                if (mine) {
#pragma unroll
                    for (int i = 0; i < PackedGroup<T>::WORDS; i++) packed.w[i] = lds[lane + i];
                }
#else
                if (mine) blend(r, base_slot, a_k, packed);
#endif
                wave_sync();  // ring rows of this step may be overwritten from here on
                STAMP(stamp); stamp++;
                if (has_next) {
                    commit_batch(nnew, slot_new, raw, ph);
                    STAMP(stamp); stamp++;
                    finish_rows(nnew, slot_new);
                    base_slot = base_slot_n;
                    a_k = a_n;
                    b_k = b_n;
                }
                // the stores of this step go out last: when the next iteration waits for its
                // prefetched loads, they have had a whole blend phase to retire
                STAMP(stamp); stamp++;
#ifdef RMX_EXP_NOSTORE
                if (mine && packed.w[0] == 0x12345678u && packed.w[1] == 0x9abcdef0u) asm_store_packed<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, x0, packed);
#else
                if (mine) asm_store_packed<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, x0, packed);
#endif
            }
        } else {
            for (int rs = r0; rs < r1; rs += G) {
                const int re = min(rs + G, r1) - 1;
                const int r = rs + lr;
                if (lane_on && r <= re) {
                    PackedGroup<T> packed;
                    blend(r, base_slot, a_k, packed);
                    store_packed<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, x0, packed);
                }
                wave_sync();
                if (rs + G < r1) {
                    const int a_n = (int)floorf(src_coord_f(pcy + rs + G, ry, offy, fylo));
                    const int b_n = (int)floorf(src_coord_f(pcy + min(rs + 2 * G, r1) - 1, ry, offy, fylo)) + 1;
                    base_slot += a_n - a_k;
                    while (base_slot >= R) base_slot -= R;
                    const int new_lo = max(b_k + 1, a_n);
                    int slot_new = base_slot + (new_lo - a_n);
                    if (slot_new >= R) slot_new -= R;
                    stage_general(new_lo, b_n - new_lo + 1, slot_new, false, !safe);
                    finish_rows(b_n - new_lo + 1, slot_new);
                    a_k = a_n;
                    b_k = b_n;
                }
            }
        }
    }
}

template <typename T, int LAYOUT>
static KernelFn pick3(bool norm, bool quant) {
    if (norm && quant) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, true>;
    if (norm) return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, true, false>;
    return (KernelFn)rmx_resize_fast_kernel<T, LAYOUT, false, false>;
}

KernelFn select_resize_fast_kernel(int dtype, int layout, bool norm, bool quant, const char **name) {
    *name = "rmx_resize_fast_kernel";
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

}  // namespace rmx
