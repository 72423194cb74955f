// K1: crop + horizontal/vertical flip + per-channel FMA + layout transpose + cast, one pass.
// Serves CropMirrorNormalize, Crop, Flip and ToTensor (u8 NHWC in; f32/f16/u8, NCHW/NHWC out).
//
// Scheduling: one wavefront owns a strip of output rows of one sample. Inside a step the
// wave covers G = 64/L rows at once, L = lanes per row, each lane producing 8 adjacent
// pixels: a 28-byte realigned read of packed RGB in, three 128-bit planar stores out (fp16).
// HBM-bound: 3 bytes read and 3*sizeof(T) written per output pixel, no reuse.
//
// FAST variant (every written width a multiple of 8, 16-byte aligned destination rows): the loads of up
// to four row steps are issued back to back before the first one is used, and the stores follow, so a
// wavefront pays one memory round trip per strip instead of one per row step (loads and stores share one
// in-order counter on this hardware: a load issued behind a store waits for that store as well).
// ANY variant of it (crops of 225, 299 ... pixels, a destination at any element): the same pipeline; the short last group of
// a row is moved left until it is whole (it then recomputes up to seven pixels of its neighbour and stores the same values to
// the same places), and a group leaves as 16-byte stores at the element's own alignment. 128 crops of 299 x 299 to fp16
// planes: 30.4 us through the general path (row by row, element-wise stores for the short group, which cost the whole
// wavefront), 22 us in this form, 20 us at 296 or 304. fp32 rows pass through the LDS slab as in the aligned form and leave as
// 16-byte pieces at 16-byte aligned addresses (60.3 -> 41.4 us; 32 us at 304). What is left of the difference belongs to the
// memory system: rows whose pitch is no multiple of a cache line share lines with their neighbours (the aligned form itself
// takes 23.0 instead of 16.7 us for 224-pixel fp32 rows at a pitch of 232).
#include "rmx_device.h"
#include "rmx_launch.h"

#ifndef RMX_K1_NT
#define RMX_K1_NT true  // streaming stores: batches larger than the last-level cache gain 13 % (20.9 against 24.1 us on the 128 x 224 x 224 fp32 batch), cache-resident replays lose 6 %
#endif

namespace rmx {

enum { CMN_GENERAL = 0, CMN_FAST = 1, CMN_FAST_ANY = 2 };

template <typename T, int LAYOUT, bool NORM, int MODE>
__global__ void __launch_bounds__(256) rmx_cmn_kernel(RmxKArgs a) {
    constexpr bool FAST = MODE != CMN_GENERAL;
    constexpr bool ANY = MODE == CMN_FAST_ANY;
    // LDS slab through which the lanes of a row exchange their runs before storing (see store_packed_coalesced)
    constexpr bool COALESCE = (MODE == CMN_FAST && coalesce_pays<T, LAYOUT>()) || (ANY && sizeof(T) == 4);
    uint32_t *slab = nullptr;
    if constexpr (COALESCE) {
        __shared__ __attribute__((aligned(16))) uint32_t slabs[4 * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>()];
        slab = slabs + (threadIdx.x / RMX_WAVE) * RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>();
    }
    const int lane = threadIdx.x & (RMX_WAVE - 1);
    const uint32_t nwaves = (uint32_t)a.n * (uint32_t)a.strips;
    uint32_t wave = xcd_swizzle(blockIdx.x, a.nblocks) * (uint32_t)a.wpb + (threadIdx.x / RMX_WAVE);
    wave = __builtin_amdgcn_readfirstlane(wave);
    if (wave >= nwaves) return;
    int s, strip;
    wave_to_sample(a, wave, s, strip);
    // whole table row in one round trip (the empty statement keeps the fetch above the early exit)
    const RmxSample P = a.table[s];
    asm volatile("" : : "s"(P.src_x), "s"(P.dst_w), "s"(P.flags), "s"(P.scale[0]), "s"(P.bias[2]));

    const int cw = P.dst_w, ch = P.dst_h;
    const int srows = a.aux0;
    const int r0 = strip * srows;
    if (r0 >= ch) return;
    const int r1 = min(r0 + srows, ch);
    const bool hf = (P.flags & RMX_S_HFLIP) != 0;
    const bool vf = (P.flags & RMX_S_VFLIP) != 0;
    const bool chrev = (P.flags & RMX_S_CHREV) != 0;
    const int x1 = P.src_x, y1 = P.src_y;

    uint32_t row_stride32;
    const uint8_t *simg = sample_base(a, s, row_stride32);
    const size_t row_stride = row_stride32;
    const uint8_t *buf_end = a.src + a.src_bytes;
    T *dimg = reinterpret_cast<T *>(a.dst) + (size_t)s * 3 * a.dst_h * a.dst_w;

    float sc[3], bi[3];
#pragma unroll
    for (int c = 0; c < 3; c++) {
        sc[c] = P.scale[c];
        bi[c] = P.bias[c];
    }

    for (int xt = 0; xt < cw; xt += RMX_WAVE * PX) {
        const int tw = min(cw - xt, RMX_WAVE * PX);
        const int L = (tw + PX - 1) / PX;  // lanes per row, <= 64
        const int G = RMX_WAVE / L;        // rows per step
        const int lr = lane / L;
        const int g = lane - lr * L;
        int gx = xt + g * PX;                     // first output column of this lane's group
        if constexpr (ANY) gx = min(gx, cw - PX);  // (the host admits this variant for rows of 8 pixels and more)
        const int cnt = min(PX, cw - gx);         // valid pixels in the group
        const bool active = lr < G;
        // source column of group pixel 0 (mirror reads the mirrored run and reverses it)
        const int sx0 = x1 + (hf ? (cw - gx - cnt) : gx);
        if constexpr (FAST) {
            // One row step of a lane: 8 pixels = 24 source bytes, fetched as a 16- and a 12-byte load from the dword below them.
            auto row_ptr = [&](int r, uint32_t &ph) {
                const int sy = y1 + (vf ? (ch - 1 - r) : r);
                const uint8_t *p = simg + (size_t)sy * row_stride + (size_t)sx0 * 3;
                ph = (uint32_t)((uintptr_t)p & 3u);
                return reinterpret_cast<const uint32_t *>(p - ph);
            };
            auto finish = [&](int r, const uint32_t (&w)[6]) {
                float v[3][PX];
                unpack8(w, v);
                if (chrev) {
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        const float t = v[0][k];
                        v[0][k] = v[2][k];
                        v[2][k] = t;
                    }
                }
                if constexpr (NORM) {
#pragma unroll
                    for (int c = 0; c < 3; c++)
#pragma unroll
                        for (int k = 0; k < PX; k++) v[c][k] = __builtin_fmaf(v[c][k], sc[c], bi[c]);
                }
                PackedGroup<T> packed;
                pack_group<T, LAYOUT>(v, hf, packed);
                if constexpr (COALESCE && ANY) store_packed_coalesced_any<T, LAYOUT, RMX_K1_NT>(slab, lane - g, g, L, min(xt, cw - PX), xt + tw - min(xt, cw - PX), dimg, a.dst_h, a.dst_w, r, gx, packed);  // (a tile narrower than 8 pixels: its one group reaches back into the tile before)
                else if constexpr (COALESCE) store_packed_coalesced<T, LAYOUT, RMX_K1_NT>(slab, lane - g, g, L, dimg, a.dst_h, a.dst_w, r, gx, packed);
                else store_packed<T, LAYOUT, RMX_K1_NT, ANY>(dimg, a.dst_h, a.dst_w, r, gx, packed);
            };
            // every wide load of this wavefront's strip stays inside the batch buffer (the first and the last row bound the rest)
            bool lane_safe = true;
            if (active) {
                uint32_t ph;
                lane_safe = (const uint8_t *)(row_ptr(r0, ph) + 7) <= buf_end && (const uint8_t *)(row_ptr(r1 - 1, ph) + 7) <= buf_end;
            }
            if (__builtin_amdgcn_ballot_w64(!lane_safe) == 0) {
                // Software pipeline over batches of NI row steps: the loads of the next batch are issued BEFORE the stores of the
                // current one. Memory operations of a wavefront complete in issue order, so the wait for a batch's loads then
                // leaves the stores of the batch before (and the loads of the batch after) outstanding: a wavefront has reads
                // and writes in flight at the same time, instead of all wavefronts of a launch reading first and writing after.
                constexpr int NI = 2;
                u32x4_a4 ta[NI], tb[NI];
                u32x3_a4 ua[NI], ub[NI];
                uint32_t pa[NI], pb[NI];
                auto issue = [&](int base, u32x4_a4 (&t)[NI], u32x3_a4 (&u)[NI], uint32_t (&ph)[NI]) {
                    if (active) {
#pragma unroll
                        for (int i = 0; i < NI; i++) {
                            const uint32_t *q = row_ptr(min(base + lr + i * G, r1 - 1), ph[i]);  // steps beyond the strip repeat its last row (never stored)
                            t[i] = *reinterpret_cast<const u32x4_a4 *>(q);
                            u[i] = *reinterpret_cast<const u32x3_a4 *>(q + 4);
                        }
                    }
                };
                auto consume = [&](int base, const u32x4_a4 (&t)[NI], const u32x3_a4 (&u)[NI], const uint32_t (&ph)[NI]) {
#pragma unroll
                    for (int i = 0; i < NI; i++) {
                        const int r = base + lr + i * G;
                        if (active && r < r1) {
                            const uint32_t d[7] = {t[i].x, t[i].y, t[i].z, t[i].w, u[i].x, u[i].y, u[i].z};
                            uint32_t w[6];
#pragma unroll
                            for (int j = 0; j < 6; j++) w[j] = __builtin_amdgcn_alignbyte(d[j + 1], d[j], ph[i]);
                            finish(r, w);
                        }
                    }
                };
                const int step = NI * G;
                issue(r0, ta, ua, pa);
                for (int base = r0; base < r1; base += 2 * step) {
                    if (base + step < r1) issue(base + step, tb, ub, pb);
                    consume(base, ta, ua, pa);
                    if (base + step < r1) {
                        if (base + 2 * step < r1) issue(base + 2 * step, ta, ua, pa);
                        consume(base + step, tb, ub, pb);
                    }
                }
            } else {
                // last bytes of the batch buffer: the bounds-checked loader, row by row
                for (int r = r0 + lr; r < r1 && active; r += G) {
                    uint32_t ph, w[6];
                    const uint32_t *q = row_ptr(r, ph);
                    load_realigned<7>(reinterpret_cast<const uint8_t *>(q) + ph, buf_end, w);
                    finish(r, w);
                }
            }
        } else {
            for (int r = r0 + lr; r < r1 && active; r += G) {
                const int sy = y1 + (vf ? (ch - 1 - r) : r);
                const uint8_t *p = simg + (size_t)sy * row_stride + (size_t)sx0 * 3;
                uint32_t w[6];
                load_realigned<7>(p, buf_end, w);
                float v[3][PX];
                unpack8(w, v);
                if (chrev) {
#pragma unroll
                    for (int k = 0; k < PX; k++) {
                        const float t = v[0][k];
                        v[0][k] = v[2][k];
                        v[2][k] = t;
                    }
                }
                if constexpr (NORM) {
#pragma unroll
                    for (int c = 0; c < 3; c++)
#pragma unroll
                        for (int k = 0; k < PX; k++) v[c][k] = __builtin_fmaf(v[c][k], sc[c], bi[c]);
                }
                store_group<T, LAYOUT>(dimg, a.dst_h, a.dst_w, r, gx, cnt, v, hf);
            }
        }
    }
}

template <typename T, int LAYOUT>
static KernelFn pick_variant(bool norm, int mode) {
    if (mode == CMN_FAST) return norm ? (KernelFn)rmx_cmn_kernel<T, LAYOUT, true, CMN_FAST> : (KernelFn)rmx_cmn_kernel<T, LAYOUT, false, CMN_FAST>;
    if (mode == CMN_FAST_ANY) return norm ? (KernelFn)rmx_cmn_kernel<T, LAYOUT, true, CMN_FAST_ANY> : (KernelFn)rmx_cmn_kernel<T, LAYOUT, false, CMN_FAST_ANY>;
    return norm ? (KernelFn)rmx_cmn_kernel<T, LAYOUT, true, CMN_GENERAL> : (KernelFn)rmx_cmn_kernel<T, LAYOUT, false, CMN_GENERAL>;
}

template <typename T>
static KernelFn pick_layout(int layout, bool norm, int mode) {
    if (layout == RMX_NCHW) return pick_variant<T, RMX_NCHW>(norm, mode);
    return pick_variant<T, RMX_NHWC>(norm, mode);
}

// mode: 0 the general kernel, 1 whole groups and 16-byte aligned destination rows, 2 rows of 8 pixels and more at any alignment
KernelFn select_cmn_kernel(int dtype, int layout, bool norm, int mode, const char **name) {
    static const char *names[3] = {"rmx_cmn_kernel<float", "rmx_cmn_kernel<__half", "rmx_cmn_kernel<unsigned char"};
    *name = names[dtype];
    switch (dtype) {
        case RMX_FP32: return pick_layout<float>(layout, norm, mode);
        case RMX_FP16: return pick_layout<__half>(layout, norm, mode);
        default: return pick_layout<uint8_t>(layout, norm, mode);
    }
}

}  // namespace rmx
