// Device-side building blocks shared by every kernel: realigned wide loads of packed RGB,
// the rounding rules, and the typed/layout-aware group stores.
#pragma once
#include "rmx_common.h"

#define RMX_DEV __device__ __forceinline__

namespace rmx {

constexpr int PX = 8;  // output pixels per lane group (8 x fp16 = one 128-bit store per channel)

// multi-dword vectors that only promise dword alignment (global memory accepts that)
typedef uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x3_a4 __attribute__((ext_vector_type(3), aligned(4)));

RMX_DEV float ubyte0(uint32_t v) { return (float)(v & 0xffu); }
RMX_DEV float ubyte1(uint32_t v) { return (float)((v >> 8) & 0xffu); }
RMX_DEV float ubyte2(uint32_t v) { return (float)((v >> 16) & 0xffu); }
RMX_DEV float ubyte3(uint32_t v) { return (float)(v >> 24); }

// u8 store rule: round-to-nearest-even, then saturate.
RMX_DEV float round_u8(float v) {
    v = __builtin_rintf(v);
    return __builtin_fminf(__builtin_fmaxf(v, 0.0f), 255.0f);
}

// First pixel and row stride (bytes) of sample s: from the layout table of a ragged source, else the padded batch.
RMX_DEV const uint8_t *sample_base(const RmxKArgs &a, int s, uint32_t &row_stride) {
    if (a.layout) {
        const RmxSrcLayout L = a.layout[s];
        row_stride = L.row_stride;
        return a.src + L.offset;
    }
    row_stride = (uint32_t)a.src_w * 3u;
    return a.src + (size_t)s * a.src_h * row_stride;
}

// Cache policy of the loads that go straight into LDS (0: default; 2: non-temporal). Non-temporal source loads were
// measured: a batch that is still in the last-level cache is then read from HBM all the same (the bilinear and triangular
// kernels run at their out-of-cache speed always, no faster out of cache), and the warp kernel, whose tiles share box rows,
// loses 7 %.
#ifndef RMX_LDS_LOAD_AUX
#define RMX_LDS_LOAD_AUX 0
#endif
typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *glb_ptr_t;
typedef __attribute__((address_space(3))) uint8_t lds_u8;    // explicit LDS pointers: every access below is a DS instruction,
typedef __attribute__((address_space(3))) uint32_t lds_u32;  // never a FLAT one (which would also count as vector memory)

// A wave-uniform value that the vector unit produced (float arithmetic has no scalar form), moved into a scalar register
// by an instruction the optimiser cannot look through: everything derived from it stays scalar arithmetic. (The
// readfirstlane builtin is folded away for values known to be uniform, and the dependants then run on the vector unit.)
// The compiler does not see inside the statement, so the wait states this chip wants around the instruction are spelled
// out: one between a vector instruction that writes the source register and the read of it, five before a vector memory
// instruction may read the scalar result (two before a vector ALU instruction may).
RMX_DEV int to_sgpr(int v) {
    int r;
    asm("s_nop 0\n\tv_readfirstlane_b32 %0, %1\n\ts_nop 4" : "=s"(r) : "v"(v));
    return r;
}

// Order LDS traffic between the lanes of one wavefront. A wave's DS instructions execute in
// issue order, so no hardware barrier is needed: this only stops the compiler from moving
// LDS reads above the writes they depend on.
RMX_DEV void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Workgroup -> XCD placement: hardware deals consecutive workgroup ids round-robin over the
// 8 XCDs (each with its own L2). Remap so that consecutive logical ids land on one XCD, which
// keeps all strips of a sample (and their shared halo rows) in a single L2.
RMX_DEV uint32_t xcd_swizzle(uint32_t b, uint32_t nblocks) {
    constexpr uint32_t XCDS = 8;
    uint32_t per = nblocks / XCDS;
    uint32_t body = per * XCDS;
    if (b >= body) return b;  // ragged tail keeps its id
    return (b % XCDS) * per + (b / XCDS);
}

// Which sample and which of its strips a wavefront works on. The launch numbers its wavefronts so that consecutive ones
// share an XCD (xcd_swizzle): XCD k gets the k-th eighth of them. Were the samples taken in batch order, a batch whose cost
// grows or falls along its length (images sorted by size) would give one XCD all the heavy samples (measured: 38 instead of
// 31 us on the RandomResizedCrop batch sorted by window area). So the samples are dealt round-robin: the i-th sample of XCD k
// is sample 8 i + k; all strips of a sample still share an XCD and its L2. The two divisions are multiplications by
// reciprocals that the host rounds up, exact for the ranges the host admits (dividend x divisor < 2^32).
// With the deal the eight XCDs also work on eight neighbouring samples at a time, one moving window of addresses instead
// of eight (measured: 2-8 % faster on uniform batches too). `deal` is false in the kernels that do not renumber their
// workgroups (xcd_swizzle): there the device already walks the batch as one stream, and a deal would only scatter it.
RMX_DEV void wave_to_sample(const RmxKArgs &a, uint32_t wave, int &sample, int &strip, bool deal = true) {
    const uint32_t strips = (uint32_t)a.strips;
    const uint32_t slot = a.inv_strips ? __umulhi(wave, a.inv_strips) : (strips == 1 ? wave : wave / strips);
    strip = (int)(wave - slot * strips);
    uint32_t s = slot;
    if (deal && slot < a.per_xcd * 8u) {
        const uint32_t k = __umulhi(slot, a.inv_per_xcd);  // slot / per_xcd: the XCD
        s = (slot - k * a.per_xcd) * 8u + k;
    }
    sample = (int)s;
}

// ---------------------------------------------------------------- source loads

// Load `ND` consecutive dwords starting at the 4-byte-aligned address that contains byte
// `p`, and realign them so that byte 0 of out[0] is *p. out has ND-1 dwords. Reads never go
// past the dword that holds the last byte of the batch buffer.
template <int ND>
RMX_DEV void load_realigned(const uint8_t *p, const uint8_t *buf_end, uint32_t (&out)[ND - 1]) {
    const uint32_t phase = (uint32_t)((uintptr_t)p & 3u);
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p - phase);  // keeps the global address space
    uint32_t d[ND];
    if ((const uint8_t *)(q + ND) <= buf_end) {
        if constexpr (ND == 4) {
            u32x4_a4 t = *reinterpret_cast<const u32x4_a4 *>(q);  // global_load_dwordx4 at dword alignment
            d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w;
        } else if constexpr (ND == 7) {
            u32x4_a4 t = *reinterpret_cast<const u32x4_a4 *>(q);
            u32x3_a4 u = *reinterpret_cast<const u32x3_a4 *>(q + 4);
            d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w; d[4] = u.x; d[5] = u.y; d[6] = u.z;
        } else {
#pragma unroll
            for (int i = 0; i < ND; i++) d[i] = q[i];
        }
    } else {
#pragma unroll
        for (int i = 0; i < ND; i++) d[i] = ((const uint8_t *)(q + i) < buf_end) ? q[i] : 0u;
    }
#pragma unroll
    for (int i = 0; i < ND - 1; i++) out[i] = __builtin_amdgcn_alignbyte(d[i + 1], d[i], phase);
}

// Split form of load_realigned<4> for software pipelining: issue the 128-bit load now, realign
// later (so that several loads can be in flight before the first use).
RMX_DEV uint32_t load_raw4(const uint8_t *p, const uint8_t *buf_end, uint32_t (&d)[4]) {
    const uint32_t phase = (uint32_t)((uintptr_t)p & 3u);
    const uint32_t *q = reinterpret_cast<const uint32_t *>(p - phase);
    if ((const uint8_t *)(q + 4) <= buf_end) {
        u32x4_a4 t = *reinterpret_cast<const u32x4_a4 *>(q);
        d[0] = t.x; d[1] = t.y; d[2] = t.z; d[3] = t.w;
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) d[i] = ((const uint8_t *)(q + i) < buf_end) ? q[i] : 0u;
    }
    return phase;
}

// raw dwords + byte phase -> 4 packed pixels expanded to one dword each (top byte is don't-care)
RMX_DEV uint4 expand4(const uint32_t (&d)[4], uint32_t phase) {
    uint32_t w0 = __builtin_amdgcn_alignbyte(d[1], d[0], phase);
    uint32_t w1 = __builtin_amdgcn_alignbyte(d[2], d[1], phase);
    uint32_t w2 = __builtin_amdgcn_alignbyte(d[3], d[2], phase);
    uint4 px;
    px.x = w0;
    px.y = __builtin_amdgcn_alignbyte(w1, w0, 3);
    px.z = __builtin_amdgcn_alignbyte(w2, w1, 2);
    px.w = w2 >> 8;
    return px;
}

// 8 packed RGB pixels (24 bytes = 6 dwords, byte 0 = R of pixel 0) -> v[c][k]
RMX_DEV void unpack8(const uint32_t (&w)[6], float (&v)[3][PX]) {
    v[0][0] = ubyte0(w[0]); v[1][0] = ubyte1(w[0]); v[2][0] = ubyte2(w[0]);
    v[0][1] = ubyte3(w[0]); v[1][1] = ubyte0(w[1]); v[2][1] = ubyte1(w[1]);
    v[0][2] = ubyte2(w[1]); v[1][2] = ubyte3(w[1]); v[2][2] = ubyte0(w[2]);
    v[0][3] = ubyte1(w[2]); v[1][3] = ubyte2(w[2]); v[2][3] = ubyte3(w[2]);
    v[0][4] = ubyte0(w[3]); v[1][4] = ubyte1(w[3]); v[2][4] = ubyte2(w[3]);
    v[0][5] = ubyte3(w[3]); v[1][5] = ubyte0(w[4]); v[2][5] = ubyte1(w[4]);
    v[0][6] = ubyte2(w[4]); v[1][6] = ubyte3(w[4]); v[2][6] = ubyte0(w[5]);
    v[0][7] = ubyte1(w[5]); v[1][7] = ubyte2(w[5]); v[2][7] = ubyte3(w[5]);
}

// ---------------------------------------------------------------- typed stores

template <typename T> struct OutCvt;
template <> struct OutCvt<float> {
    static RMX_DEV float cvt(float v) { return v; }
};
template <> struct OutCvt<__half> {
    // The value passes through an empty statement first: the compiler would otherwise merge the conversion
    // into an FMA that produces it (v_fma_mixlo_f16), which rounds the exact sum to fp16 once, where the
    // reference rounds to fp32 and then to fp16; the two differ in about one value in 40 000.
    static RMX_DEV __half cvt(float v) {
        asm("" : "+v"(v));
        return __float2half_rn(v);
    }
};
template <> struct OutCvt<uint8_t> {
    static RMX_DEV uint8_t cvt(float v) { return (uint8_t)round_u8(v); }
};

template <int ALIGN> struct ElemAligned;  // 16-, 8- and 4-byte values at the alignment of a 1-, 2- or 4-byte element
template <> struct ElemAligned<1> {
    typedef uint32_t x4 __attribute__((ext_vector_type(4), aligned(1)));
    typedef uint32_t x2 __attribute__((ext_vector_type(2), aligned(1)));
    typedef uint32_t x1 __attribute__((aligned(1)));
};
template <> struct ElemAligned<2> {
    typedef uint32_t x4 __attribute__((ext_vector_type(4), aligned(2)));
    typedef uint32_t x2 __attribute__((ext_vector_type(2), aligned(2)));
    typedef uint32_t x1 __attribute__((aligned(2)));
};
template <> struct ElemAligned<4> {
    typedef uint32_t x4 __attribute__((ext_vector_type(4), aligned(4)));
    typedef uint32_t x2 __attribute__((ext_vector_type(2), aligned(4)));
    typedef uint32_t x1 __attribute__((aligned(4)));
};
// Store `cnt` (<= N) consecutive elements. A full run leaves as 128/64/32-bit stores at whatever alignment the element type
// gives its address (vector memory instructions take any address on this target; a run that straddles a cache line is split
// by the hardware), a partial one element by element. Measured on 256 images resized to 225 x 225 fp16 planes, where odd rows
// start at odd multiples of 2 bytes: 59.9 -> 47.8 us against a ladder of alignment tests that ended in element-wise stores
// (interleaved fp16 at 227 x 227: 82.7 -> 47.3 us).
// NT: streaming (non-temporal) stores.
template <typename T>
RMX_DEV void store_elem_nt(T *p, T v) {
    if constexpr (sizeof(T) == 4) __builtin_nontemporal_store(__builtin_bit_cast(uint32_t, v), reinterpret_cast<uint32_t *>(p));
    else if constexpr (sizeof(T) == 2) __builtin_nontemporal_store(__builtin_bit_cast(uint16_t, v), reinterpret_cast<uint16_t *>(p));
    else __builtin_nontemporal_store((uint8_t)v, reinterpret_cast<uint8_t *>(p));
}
template <typename T, int N, bool NT = false>
RMX_DEV void store_run(T *p, const T (&e)[N], int cnt) {
    constexpr int BYTES = N * (int)sizeof(T);
    typedef typename ElemAligned<(int)sizeof(T)>::x4 u32x4_e;
    typedef typename ElemAligned<(int)sizeof(T)>::x2 u32x2_e;
    typedef typename ElemAligned<(int)sizeof(T)>::x1 u32x1_e;
    if (cnt == N) {
        if constexpr (BYTES % 16 == 0) {
            u32x4_e t[BYTES / 16];
            __builtin_memcpy(t, e, BYTES);
#pragma unroll
            for (int i = 0; i < BYTES / 16; i++) {
                if constexpr (NT) __builtin_nontemporal_store(t[i], reinterpret_cast<u32x4_e *>(p) + i);
                else reinterpret_cast<u32x4_e *>(p)[i] = t[i];
            }
            return;
        } else if constexpr (BYTES % 8 == 0) {
            u32x2_e t[BYTES / 8];
            __builtin_memcpy(t, e, BYTES);
#pragma unroll
            for (int i = 0; i < BYTES / 8; i++) {
                if constexpr (NT) __builtin_nontemporal_store(t[i], reinterpret_cast<u32x2_e *>(p) + i);
                else reinterpret_cast<u32x2_e *>(p)[i] = t[i];
            }
            return;
        } else if constexpr (BYTES % 4 == 0) {
            u32x1_e t[BYTES / 4];
            __builtin_memcpy(t, e, BYTES);
#pragma unroll
            for (int i = 0; i < BYTES / 4; i++) reinterpret_cast<u32x1_e *>(p)[i] = t[i];
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < N; i++)
        if (i < cnt) {
            if constexpr (NT) store_elem_nt<T>(p + i, e[i]);
            else p[i] = e[i];
        }
}

// Full-group store for callers that have established alignment: N*sizeof(T) is a multiple of 8
// and p is aligned to min(16, N*sizeof(T) & -N*sizeof(T)) bytes.
template <typename T, int N>
RMX_DEV void store_run_aligned(T *p, const T (&e)[N]) {
    constexpr int BYTES = N * (int)sizeof(T);
    if constexpr (BYTES % 16 == 0) {
        uint4 t[BYTES / 16];
        __builtin_memcpy(t, e, BYTES);
#pragma unroll
        for (int i = 0; i < BYTES / 16; i++) reinterpret_cast<uint4 *>(p)[i] = t[i];
    } else {
        static_assert(BYTES % 8 == 0, "group must be a multiple of 8 bytes");
        uint2 t[BYTES / 8];
        __builtin_memcpy(t, e, BYTES);
#pragma unroll
        for (int i = 0; i < BYTES / 8; i++) reinterpret_cast<uint2 *>(p)[i] = t[i];
    }
}

// Full, aligned group of PX pixels (see store_group for the meaning of rev).
template <typename T, int LAYOUT>
RMX_DEV void store_group_aligned(T *sample, int H, int W, int y, int x0, const float (&v)[3][PX], bool rev) {
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T e[PX];
#pragma unroll
            for (int k = 0; k < PX; k++) e[k] = OutCvt<T>::cvt(rev ? v[c][PX - 1 - k] : v[c][k]);
            store_run_aligned<T, PX>(sample + ((size_t)c * H + y) * W + x0, e);
        }
    } else {
        T e[PX * 3];
#pragma unroll
        for (int k = 0; k < PX; k++)
#pragma unroll
            for (int c = 0; c < 3; c++) e[k * 3 + c] = OutCvt<T>::cvt(rev ? v[c][PX - 1 - k] : v[c][k]);
        store_run_aligned<T, PX * 3>(sample + ((size_t)y * W + x0) * 3, e);
    }
}

// Split form of store_group_aligned: pack now (values become PX*3*sizeof(T) bytes of registers in
// memory order), store later. Lets a kernel keep finished pixels in few registers while other
// memory operations complete.
template <typename T>
struct PackedGroup {
    static constexpr int WORDS = PX * 3 * (int)sizeof(T) / 4;
    uint32_t w[WORDS];
};

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <typename T, int LAYOUT, bool REV>
RMX_DEV void pack_group_dir(const float (&v)[3][PX], PackedGroup<T> &out) {
    if constexpr (sizeof(T) == 2) {
        // fp16: two values per conversion (round-to-nearest-even, as __float2half_rn)
#pragma unroll
        for (int i = 0; i < PX * 3 / 2; i++) {
            float lo, hi;
            if constexpr (LAYOUT == RMX_NCHW) {
                const int c = (2 * i) / PX, k = (2 * i) % PX;
                lo = REV ? v[c][PX - 1 - k] : v[c][k];
                hi = REV ? v[c][PX - 2 - k] : v[c][k + 1];
            } else {
                const int k0 = (2 * i) / 3, c0 = (2 * i) % 3, k1 = (2 * i + 1) / 3, c1 = (2 * i + 1) % 3;
                lo = REV ? v[c0][PX - 1 - k0] : v[c0][k0];
                hi = REV ? v[c1][PX - 1 - k1] : v[c1][k1];
            }
            const f16x2 h = __builtin_convertvector((f32x2){lo, hi}, f16x2);
            __builtin_memcpy(&out.w[i], &h, 4);
        }
        return;
    }
    if constexpr (sizeof(T) == 1) {
        // u8: v_cvt_pk_u8_f32 rounds to nearest even, saturates to 0..255 and drops the byte into place
#pragma unroll
        for (int i = 0; i < PX * 3 / 4; i++) {
            uint32_t w = 0;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int e = 4 * i + b;
                float val;
                if constexpr (LAYOUT == RMX_NCHW) {
                    const int c = e / PX, k = e % PX;
                    val = REV ? v[c][PX - 1 - k] : v[c][k];
                } else {
                    const int k = e / 3, c = e % 3;
                    val = REV ? v[c][PX - 1 - k] : v[c][k];
                }
                w = __builtin_amdgcn_cvt_pk_u8_f32(val, b, w);
            }
            out.w[i] = w;
        }
        return;
    }
    T e[PX * 3];
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++)
#pragma unroll
            for (int k = 0; k < PX; k++) e[c * PX + k] = OutCvt<T>::cvt(REV ? v[c][PX - 1 - k] : v[c][k]);
    } else {
#pragma unroll
        for (int k = 0; k < PX; k++)
#pragma unroll
            for (int c = 0; c < 3; c++) e[k * 3 + c] = OutCvt<T>::cvt(REV ? v[c][PX - 1 - k] : v[c][k]);
    }
    __builtin_memcpy(out.w, e, sizeof(e));
}

// rev is wave-uniform (one sample per wave): branch once instead of selecting per element
template <typename T, int LAYOUT>
RMX_DEV void pack_group(const float (&v)[3][PX], bool rev, PackedGroup<T> &out) {
    if (rev) pack_group_dir<T, LAYOUT, true>(v, out);
    else pack_group_dir<T, LAYOUT, false>(v, out);
}

typedef uint32_t u32x4_v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_v __attribute__((ext_vector_type(2)));
// 16- and 8-byte stores; NT = streaming (non-temporal). Measured on MI355X at steady clocks: streaming stores take
// 1.3-1.5 us off the fp16 output of the bilinear fast path (31.3 -> 29.8 us) and off the u8 output of the colour kernel
// (24.3 -> 23.0 us), change nothing for the warp kernel and cost 5-10 us on fp32 outputs, so only those two use them.
// EA = 0: the address is aligned to the store's size; 1, 2, 4: only to an element of that many bytes.
template <bool NT, int EA = 0>
RMX_DEV void st4(void *p, uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
    if constexpr (EA != 0) {
        typedef typename ElemAligned<EA>::x4 vec;
        const vec t = {a, b, c, d};
        if constexpr (NT) __builtin_nontemporal_store(t, reinterpret_cast<vec *>(p));
        else *reinterpret_cast<vec *>(p) = t;
    } else if constexpr (NT) __builtin_nontemporal_store((u32x4_v){a, b, c, d}, reinterpret_cast<u32x4_v *>(p));
    else *reinterpret_cast<uint4 *>(p) = make_uint4(a, b, c, d);
}
template <bool NT, int EA = 0>
RMX_DEV void st2(void *p, uint32_t a, uint32_t b) {
    if constexpr (EA != 0) {
        typedef typename ElemAligned<EA>::x2 vec;
        const vec t = {a, b};
        if constexpr (NT) __builtin_nontemporal_store(t, reinterpret_cast<vec *>(p));
        else *reinterpret_cast<vec *>(p) = t;
    } else if constexpr (NT) __builtin_nontemporal_store((u32x2_v){a, b}, reinterpret_cast<u32x2_v *>(p));
    else *reinterpret_cast<uint2 *>(p) = make_uint2(a, b);
}

// ANY: the run may start at any element (else: at a multiple of its store size).
template <typename T, int LAYOUT, bool NT = false, bool ANY = false>
RMX_DEV void store_packed(T *sample, int H, int W, int y, int x0, const PackedGroup<T> &g) {
    constexpr int PW = PX * (int)sizeof(T) / 4;  // dwords per channel run
    constexpr int EA = ANY ? (int)sizeof(T) : 0;
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T *p = sample + ((size_t)c * H + y) * W + x0;
            if constexpr (PW % 4 == 0) {
#pragma unroll
                for (int i = 0; i < PW / 4; i++)
                    st4<NT, EA>(reinterpret_cast<char *>(p) + 16 * i, g.w[c * PW + 4 * i], g.w[c * PW + 4 * i + 1], g.w[c * PW + 4 * i + 2], g.w[c * PW + 4 * i + 3]);
            } else {
#pragma unroll
                for (int i = 0; i < PW / 2; i++) st2<NT, EA>(reinterpret_cast<char *>(p) + 8 * i, g.w[c * PW + 2 * i], g.w[c * PW + 2 * i + 1]);
            }
        }
    } else {
        T *p = sample + ((size_t)y * W + x0) * 3;
        constexpr int TW = PackedGroup<T>::WORDS;
        if constexpr (TW % 4 == 0) {
#pragma unroll
            for (int i = 0; i < TW / 4; i++) st4<NT, EA>(reinterpret_cast<char *>(p) + 16 * i, g.w[4 * i], g.w[4 * i + 1], g.w[4 * i + 2], g.w[4 * i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < TW / 2; i++) st2<NT, EA>(reinterpret_cast<char *>(p) + 8 * i, g.w[2 * i], g.w[2 * i + 1]);
        }
    }
}

// Coalescing form of store_packed for the layouts in which a lane's run is longer than one store: fp32 planes (32 bytes per lane
// and plane) and every interleaved layout (24 / 48 / 96 bytes per lane). Stored directly, each instruction of the wavefront
// writes 16 (or 8) bytes out of every 32 .. 96, so every cache line is written by several instructions, each with part of it.
// Here the L lanes that share a destination row pass their runs through the wavefront's LDS slab and every instruction
// writes one contiguous piece of the row: chunk j of lane l is the (j*L + l)-th chunk of the row segment.
//   slab : wavefront-private LDS, RMX_WAVE * coalesce_slab_dwords<T, LAYOUT>() dwords;  grp0 : first lane of the row group;
//   pos, L : place of this lane's run in the row (ascending columns; differs from the lane order when a kernel mirrors by
//   reversing its lanes), lanes per row.
// Lanes of one row group must call it together (they do: a group shares its row and its loop conditions).
template <typename T, int LAYOUT>
constexpr int coalesce_slab_dwords() {
    return LAYOUT == RMX_NCHW ? PX * (int)sizeof(T) / 4 : PX * 3 * (int)sizeof(T) / 4;
}
// Measured on MI355X (CropMirrorNormalize 256x256 -> 224x224, batch 128, direct -> coalesced): fp32 planar 18.3 -> 15.6 us,
// fp32 interleaved 28.5 -> 15.8 us, fp16 interleaved 14.9 -> 10.5 us; u8 interleaved (8-byte chunks) gains nothing and
// fp16 / u8 planar runs are one store per lane already.
template <typename T, int LAYOUT>
constexpr bool coalesce_pays() {
    return sizeof(T) == 4 || (LAYOUT == RMX_NHWC && sizeof(T) == 2);
}

template <int W, int CH, bool NT>
RMX_DEV void store_run_coalesced(uint32_t *slab, uint8_t *seg, int grp0, int l, int L, const uint32_t *w) {
    uint32_t *mine = slab + (grp0 + l) * W;
#pragma unroll
    for (int j = 0; j < W / CH; j++) {
        if constexpr (CH == 4) *reinterpret_cast<uint4 *>(mine + 4 * j) = make_uint4(w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]);
        else *reinterpret_cast<uint2 *>(mine + 2 * j) = make_uint2(w[2 * j], w[2 * j + 1]);
    }
    wave_sync();
    const uint32_t *grp = slab + grp0 * W;
#pragma unroll
    for (int j = 0; j < W / CH; j++) {
        const int idx = (j * L + l) * CH;
        if constexpr (CH == 4) {
            const uint4 v = *reinterpret_cast<const uint4 *>(grp + idx);
            st4<NT>(seg + (size_t)idx * 4, v.x, v.y, v.z, v.w);
        } else {
            const uint2 v = *reinterpret_cast<const uint2 *>(grp + idx);
            st2<NT>(seg + (size_t)idx * 4, v.x, v.y);
        }
    }
    wave_sync();  // the slab is reused by the next call
}

// x0 is the first destination column of this lane's run; the row group's segment starts `pos` runs to the left of it.
template <typename T, int LAYOUT, bool NT = false>
RMX_DEV void store_packed_coalesced(uint32_t *slab, int grp0, int pos, int L, T *sample, int H, int W, int y, int x0, const PackedGroup<T> &g) {
    constexpr int PW = PX * (int)sizeof(T) / 4;  // dwords per channel run
    const int l = pos;
    const int xs = x0 - pos * PX;                // first column of the row group
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T *seg = sample + ((size_t)c * H + y) * W + xs;
            store_run_coalesced<PW, (PW % 4 == 0) ? 4 : 2, NT>(slab, reinterpret_cast<uint8_t *>(seg), grp0, l, L, &g.w[c * PW]);
        }
    } else {
        constexpr int TW = PackedGroup<T>::WORDS;
        T *seg = sample + ((size_t)y * W + xs) * 3;
        store_run_coalesced<TW, (TW % 4 == 0) ? 4 : 2, NT>(slab, reinterpret_cast<uint8_t *>(seg), grp0, l, L, g.w);
    }
}

// The same for fp32 rows of any width at any (4-byte) alignment, whose last run overlaps its neighbour: a lane's run of W
// dwords goes to the slab at its own offset `off` (dwords) in the row group's segment of `total` dwords, overlapping runs
// writing the same values; the segment then leaves as 16-byte pieces at 16-byte aligned addresses, consecutive lanes writing
// consecutive pieces (the slab is read at the matching, dword-aligned offset), and the up to three dwords in front of the
// first piece and behind the last one by one. (16-byte stores at addresses that are only dword-aligned were measured as slow
// as no exchange at all: 128 crops of 225 x 225 to fp32 planes 27.1 us either way.)
template <int W, bool NT>
RMX_DEV void store_run_coalesced_any(uint32_t *slab, uint8_t *seg, int grp0, int l, int L, int off, int total, const uint32_t *w) {
    typedef typename ElemAligned<4>::x4 vec;
    uint32_t *grp = slab + grp0 * W;
#pragma unroll
    for (int j = 0; j < W / 4; j++) *reinterpret_cast<vec *>(grp + off + 4 * j) = (vec){w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]};
    wave_sync();
    const int head = min((int)((4u - (uint32_t)(((uintptr_t)seg >> 2) & 3u)) & 3u), total);  // dwords in front of the first aligned piece
    const int body = (total - head) >> 2;                                                   // aligned pieces
    for (int idx = l; idx < body; idx += L) {
        const vec v = *reinterpret_cast<const vec *>(grp + head + 4 * idx);
        st4<NT>(seg + (size_t)(head + 4 * idx) * 4, v.x, v.y, v.z, v.w);
    }
    const int loose = total - 4 * body;  // head + tail, at most six dwords
    for (int e = l; e < loose; e += L) {
        const int i = e < head ? e : 4 * body + e;
        reinterpret_cast<uint32_t *>(seg)[i] = grp[i];
    }
    wave_sync();  // the slab is reused by the next call
}

// xs: first column of the row group, tw: its width in pixels; x0: first column of this lane's run (fp32 only).
template <typename T, int LAYOUT, bool NT = false>
RMX_DEV void store_packed_coalesced_any(uint32_t *slab, int grp0, int l, int L, int xs, int tw, T *sample, int H, int W, int y, int x0, const PackedGroup<T> &g) {
    static_assert(sizeof(T) == 4, "runs of whole dwords per pixel");
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T *seg = sample + ((size_t)c * H + y) * W + xs;
            store_run_coalesced_any<PX, NT>(slab, reinterpret_cast<uint8_t *>(seg), grp0, l, L, x0 - xs, tw, &g.w[c * PX]);
        }
    } else {
        T *seg = sample + ((size_t)y * W + xs) * 3;
        store_run_coalesced_any<PX * 3, NT>(slab, reinterpret_cast<uint8_t *>(seg), grp0, l, L, 3 * (x0 - xs), 3 * tw, g.w);
    }
}

// Write one lane's group of N horizontally adjacent pixels (v[c][k], k-th pixel of the group)
// to output row y starting at column x0. `cnt` pixels are valid. When `rev` the group is
// written in reversed pixel order (horizontal mirror): pixel k goes to column x0 + cnt-1-k.
template <typename T, int LAYOUT, int N = PX, bool NT = false>
RMX_DEV void store_group(T *sample, int H, int W, int y, int x0, int cnt, const float (&v)[3][N], bool rev) {
    if (cnt <= 0) return;
    if constexpr (LAYOUT == RMX_NCHW) {
#pragma unroll
        for (int c = 0; c < 3; c++) {
            T e[N];
            if (rev && cnt == N) {
#pragma unroll
                for (int k = 0; k < N; k++) e[k] = OutCvt<T>::cvt(v[c][N - 1 - k]);
            } else if (rev) {
#pragma unroll
                for (int k = 0; k < N; k++) {
                    float s = v[c][0];
#pragma unroll
                    for (int j = 1; j < N; j++) s = (j == cnt - 1 - k) ? v[c][j] : s;
                    e[k] = OutCvt<T>::cvt(s);
                }
            } else {
#pragma unroll
                for (int k = 0; k < N; k++) e[k] = OutCvt<T>::cvt(v[c][k]);
            }
            T *p = sample + ((size_t)c * H + y) * W + x0;
            store_run<T, N, NT>(p, e, cnt);
        }
    } else {
        T e[N * 3];
        if (rev && cnt == N) {
#pragma unroll
            for (int k = 0; k < N; k++)
#pragma unroll
                for (int c = 0; c < 3; c++) e[k * 3 + c] = OutCvt<T>::cvt(v[c][N - 1 - k]);
        } else if (rev) {
#pragma unroll
            for (int k = 0; k < N; k++)
#pragma unroll
                for (int c = 0; c < 3; c++) {
                    float s = v[c][0];
#pragma unroll
                    for (int j = 1; j < N; j++) s = (j == cnt - 1 - k) ? v[c][j] : s;
                    e[k * 3 + c] = OutCvt<T>::cvt(s);
                }
        } else {
#pragma unroll
            for (int k = 0; k < N; k++)
#pragma unroll
                for (int c = 0; c < 3; c++) e[k * 3 + c] = OutCvt<T>::cvt(v[c][k]);
        }
        T *p = sample + ((size_t)y * W + x0) * 3;
        store_run<T, N * 3, NT>(p, e, cnt * 3);
    }
}

}  // namespace rmx
