// Shared host/device definitions of the MI355X augmentation library: the per-sample row of
// the per-batch parameter table, kernel launch arguments and host-side bookkeeping.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/rocal_mi355x.h"

// One row per sample; the whole batch's table is uploaded once per update and every
// workgroup reads its sample's row with scalar loads (the row index is wave-uniform).
struct __attribute__((aligned(16))) RmxSample {
    int32_t src_x, src_y, src_w, src_h;  // source window in pixels (ROI or crop), XYWH
    int32_t dst_w, dst_h;                // valid output size written for this sample
    int32_t pc_x, pc_y;                  // offset of the written window inside the virtual resized image
    int32_t rs_w, rs_h;                  // virtual resized size (== dst when there is no post-crop)
    uint32_t flags;                      // RMX_S_*
    int32_t strip_rows;                  // output rows per wave strip for this sample
    float rx, ry;                        // src_len / rs_len (IEEE division done on the host)
    float fsx, fsy;                      // triangular: ratio > 1 ? 1/ratio : 1
    float scale[3], bias[3];             // normalisation: out = v*scale + bias
    union {
        float color[4];                  // colour twist: alpha, beta, hue shift in sextants [0,6], saturation
        int32_t plan[4];                 // bilinear fast paths: x-tile width for this sample, [0] staged kernel, [1] streaming kernel
    };
    float m[6];                          // warp: destination -> source affine about the centres
};
static_assert(sizeof(RmxSample) == 128, "parameter table row must stay 128 bytes");

// Where a sample's image lies when the source is not one padded [N,Hmax,Wmax,3] tensor: tightly packed images of
// different sizes, one after the other (or anywhere) in one buffer.
struct RmxSrcLayout {
    uint64_t offset;      // bytes from the source base to the sample's first pixel
    uint32_t row_stride;  // bytes per image row
    uint32_t rows;        // image height
};
static_assert(sizeof(RmxSrcLayout) == 16, "source layout entry must stay 16 bytes");

enum : uint32_t {
    RMX_S_HFLIP = 1u,
    RMX_S_VFLIP = 2u,
    RMX_S_CHREV = 4u,    // output channel k reads source channel 2-k
    RMX_S_EDGE_REF = 8u  // bilinear: both neighbours clamp to the window's last-but-one column / row (RMX_F_EDGE_REF)
};

struct RmxKArgs {
    const uint8_t *src;      // batch base, u8 NHWC
    void *dst;               // batch base
    const RmxSample *table;  // device table, n rows
    uint64_t src_bytes;      // total bytes of the source batch (bounds the wide loads)
    int32_t n;
    int32_t src_h, src_w;    // padded source dims (pixels); row stride = src_w*3
    int32_t dst_h, dst_w;    // padded destination dims
    int32_t strips;          // wave strips per sample (grid = n*strips waves)
    int32_t lds_bytes;       // dynamic LDS per wave
    int32_t aux0, aux1;
    int32_t wpb;             // wavefronts per workgroup of this launch
    uint32_t nblocks;        // workgroups of this launch
    const RmxSrcLayout *layout;  // per-sample source placement, or null: sample s starts at s*src_h*src_w*3
    const uint8_t *src2;         // second source batch of the same shape (Blend), else null
    const uint8_t *extra;        // per-sample side table behind the layout entries (Gamma: 256 bytes per sample), else null
    // wavefront -> (sample, strip) without a division, and samples dealt round-robin to the XCDs (see wave_to_sample)
    uint32_t inv_strips;         // ceil(2^32 / strips), or 0: divide
    uint32_t per_xcd, inv_per_xcd;  // samples per XCD (n / 8) and ceil(2^32 / per_xcd); per_xcd 0: samples in batch order
};

#define RMX_WAVE 64

// Hue shift of a sample in sextants (ColorTwist, Hue, Saturation). A pixel's hue before it is brought back into [0, 6] lies in
// [shift - 1.0000002, shift + 5.0000002]; below RMX_HUE_SHIFT_LOW it can never reach 6, from RMX_HUE_SHIFT_HIGH on never fall
// below 0, and one comparison brings it back. The host picks the twist kernel with the single comparison for batches in
// which every sample's shift is on one side or the other; the kernel tells the sides apart with the same comparison.
#define RMX_HUE_SHIFT_LOW 0.99998f
#define RMX_HUE_SHIFT_HIGH 1.00002f
