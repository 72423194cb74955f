/*
 * rocal_mi355x.h - C ABI of the MI355X (gfx950) augmentation hot path for rocAL.
 *
 * Every entry point is extern "C" and takes plain pointers, sizes and PODs only. The protocol
 * follows rocAL's three phases for a node:
 *
 *   create   (Node::create_node, user thread, once)        -> rmx_create_<op>()
 *   update   (Node::update_node, output thread, per batch) -> rmx_update_<op>()  [host arrays in]
 *   process  (Graph::process = vxProcessGraph, per batch)  -> rmx_op_launch()    [device buffers]
 *
 * rmx_update_* packs the per-sample host arrays (the vx_arrays / ROI tensors of the reference)
 * into one row of a per-batch parameter table and uploads it asynchronously on the context's
 * stream; rmx_op_launch() enqueues ONE kernel that covers the whole ragged batch. Nothing
 * blocks except rmx_ctx_sync(). All functions return 0 on success or an rmx_status code;
 * rmx_last_error() returns the message of the calling thread's last failure.
 *
 * Image batches use rocAL's dense tensor model (rocAL/source/pipeline/tensor.cpp:116-137):
 * [N, Hmax, Wmax, C] (NHWC) or [N, C, Hmax, Wmax] (NCHW), sample i valid inside its ROI.
 */
#ifndef ROCAL_MI355X_H
#define ROCAL_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RMX_API __attribute__((visibility("default")))

typedef struct rmx_ctx rmx_ctx;
typedef struct rmx_op rmx_op;

enum rmx_status {
    RMX_OK = 0,
    RMX_ERR_INVALID = 1,     /* bad argument (message says which) */
    RMX_ERR_HIP = 2,         /* a HIP runtime call failed (message carries the numeric code) */
    RMX_ERR_UNSUPPORTED = 3, /* combination outside the hot path (e.g. cubic interpolation) */
    RMX_ERR_NOMEM = 4
};

/* rocAL/include/pipeline/commons.h:45-70,110-113 */
enum { RMX_NHWC = 0, RMX_NCHW = 1 };
enum { RMX_FP32 = 0, RMX_FP16 = 1, RMX_UINT8 = 2 };
enum { RMX_ROI_LTRB = 0, RMX_ROI_XYWH = 1 };
/* rocAL/include/api/rocal_api_types.h:347-366 */
enum { RMX_INTERP_NEAREST = 0, RMX_INTERP_LINEAR = 1, RMX_INTERP_TRIANGULAR = 5 };

/* flags for resize-family ops */
enum {
    RMX_F_QUANTIZE_U8 = 1u << 0, /* round the resampled value to u8 before normalising: reproduces the
                                    two-node graph resize(u8) -> CropMirrorNormalize in one pass */
    /* one colour node between the resize and the CropMirrorNormalize stage of a fused chain (bilinear, with
     * RMX_F_QUANTIZE_U8): reproduces the three-node graph resize(u8) -> colour(u8) -> CropMirrorNormalize in one pass,
     * the colour node's rounded, saturated u8 output included. Parameters come with rmx_update_resize_color_cmn. */
    RMX_F_COLOR_LINEAR = 1u << 1, /* Brightness / Contrast / Exposure: fma(x - c2, c0, c1) */
    RMX_F_COLOR_TWIST = 1u << 2,  /* ColorTwist / Hue / Saturation: c0 alpha, c1 beta, c2 hue in degrees, c3 saturation */
    /* Bilinear edge rule of the reference's device code (rocAL/rocAL_hip/rocal_hip_kernels.cpp:340-343,356-361): BOTH
     * neighbours of a tap are clamped to [lo, hi-1], so the window's last column and row are never sampled; ratio, offsets
     * and weights still come from the full window length. Without the flag the neighbours clamp to [lo, hi] (the textbook
     * half-pixel-centre form, which torch.nn.functional.interpolate also computes). */
    RMX_F_EDGE_REF = 1u << 3
};

/* TensorInfo of one side of a node (rocAL/include/pipeline/tensor.h:65-309): padded maxima. */
typedef struct rmx_tensor_desc {
    uint32_t n, h, w, c;
    int32_t layout; /* RMX_NHWC | RMX_NCHW */
    int32_t dtype;  /* RMX_FP32 | RMX_FP16 | RMX_UINT8 */
} rmx_tensor_desc;

/* ---- context: one device + one stream (rocAL/source/device/device_manager_hip.cpp:53-77) ---- */
/* own_stream != 0: the context creates (and later destroys) its own non-blocking stream and
 * `stream` is ignored. own_stream == 0: `stream` is a hipStream_t to borrow (NULL = the device's
 * default stream). */
RMX_API int rmx_ctx_create(int device, void *stream, int own_stream, rmx_ctx **out);
/* Destroying a context that still has ops is allowed: the context's streams live on until the last of its ops is destroyed. */
RMX_API int rmx_ctx_destroy(rmx_ctx *ctx);
RMX_API int rmx_ctx_sync(rmx_ctx *ctx);
RMX_API void *rmx_ctx_stream(rmx_ctx *ctx);
RMX_API const char *rmx_last_error(void);
RMX_API const char *rmx_version(void);

/* ---- process: replaces vxProcessGraph for one node (rocAL/source/pipeline/graph.cpp:96-103) ---- */
/* src/dst are device pointers to the batch buffers, borrowed for the duration of the kernel
 * (rocAL swaps them every batch, rocAL/source/pipeline/tensor.cpp:478-489). Asynchronous. */
RMX_API int rmx_op_launch(rmx_op *op, const void *src, void *dst);
RMX_API int rmx_op_destroy(rmx_op *op);
/* Ragged source: instead of one padded [N,Hmax,Wmax,3] tensor the images of a batch lie tightly packed (row stride =
 * width*3) at byte `offsets[i]` of ONE device buffer of `buffer_bytes`, each with its own `widths[i]` x `heights[i]`
 * (<= the w x h of the source descriptor, which then only bounds the sizes). ROIs of later updates are relative to each
 * image. Takes effect with the next rmx_update_* of the op and stays until called again; all three arrays NULL go
 * back to the padded tensor. Stands where rocAL copies every decoded image into the padded batch
 * (rocAL/source/loaders/image/image_read_and_decode.cpp:165-390, circular_buffer.cpp:88-133): a C1 batch is
 * 315 MB padded for about 80 MB of pixels. */
RMX_API int rmx_op_set_ragged_source(rmx_op *op, const uint64_t *offsets, const uint32_t *widths, const uint32_t *heights, uint64_t buffer_bytes);
/* The same with a row stride per image (bytes, >= width*3; NULL: width*3). A loader that starts every image at a multiple of 4
 * bytes and pads its rows to a multiple of 4 bytes gives the bilinear resize its streaming kernel (source rows straight into
 * LDS), which needs every row of the batch to start at the same byte phase; the padding is at most 3 bytes per row. */
RMX_API int rmx_op_set_ragged_source_strided(rmx_op *op, const uint64_t *offsets, const uint32_t *widths, const uint32_t *heights,
                                             const uint32_t *row_strides, uint64_t buffer_bytes);
/* Algorithmic bytes of the last update: sum of source-window bytes + destination bytes. */
RMX_API uint64_t rmx_op_algorithmic_bytes(const rmx_op *op);
/* Launch plan of the last update as text (waves, strips, LDS per wave ...), for logs and benchmarks. */
RMX_API const char *rmx_op_plan(const rmx_op *op);
/* Name of the kernel the op launches (as it appears in a rocprofv3 kernel trace). */
RMX_API const char *rmx_op_kernel_name(const rmx_op *op);

/* ---- CropMirrorNormalize: replaces vxExtRppCropMirrorNormalize
 *      (rocAL/source/augmentations/geometry_augmentations/node_crop_mirror_normalize.cpp:87-88).
 * out[n,c,y,x] = in[n, y1+y, x1+(mirror? cw-1-x : x), c] * scale[n*C+c] + bias[n*C+c] (one fp32 FMA).
 * rocAL passes bias in its "multiplier" array and scale in its "offset" array (:56-61). */
RMX_API int rmx_create_crop_mirror_normalize(rmx_ctx *ctx, const rmx_tensor_desc *src,
                                             const rmx_tensor_desc *dst, int roi_type, rmx_op **out);
RMX_API int rmx_update_crop_mirror_normalize(rmx_op *op, const uint32_t *crop_roi /*[N][4]*/,
                                             const float *scale /*[N*C]*/, const float *bias /*[N*C]*/,
                                             const uint32_t *mirror /*[N]*/);

/* ---- Crop: replaces vxExtRppCrop (node_crop.cpp:47-48, node_random_crop.cpp:47) ---- */
RMX_API int rmx_create_crop(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                            int roi_type, rmx_op **out);
RMX_API int rmx_update_crop(rmx_op *op, const uint32_t *crop_roi);

/* ---- Flip: replaces vxExtRppFlip (node_flip.cpp:44-45) ---- */
RMX_API int rmx_create_flip(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                            int roi_type, rmx_op **out);
RMX_API int rmx_update_flip(rmx_op *op, const uint32_t *src_roi, const uint32_t *horizontal,
                            const uint32_t *vertical);

/* ---- ToTensor: replaces the second normalise/transpose/cast pass MasterGraph::to_tensor runs on a u8 output
 *      (rocAL/source/pipeline/master_graph.cpp:514-856) and its device kernels Hip_CopyInt8ToNCHW/NHWC
 *      (rocAL/rocAL_hip/rocal_hip_kernels.cpp:40-308): out[n,k,y,x] = fmaf(in[n,y,x,rev? 2-k : k],
 *      multiplier[k], offset[k]) over the whole padded image. multiplier and offset hold 3 floats. ---- */
RMX_API int rmx_create_to_tensor(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, rmx_op **out);
RMX_API int rmx_update_to_tensor(rmx_op *op, const float *multiplier /*[3]*/, const float *offset /*[3]*/, int reverse_channels);

/* ---- Resize family: replaces vxExtRppResize (node_resize.cpp:56-57, node_crop_resize.cpp:60-61),
 *      vxExtRppResizeCropMirror (node_resize_crop_mirror.cpp:59-60) and
 *      vxExtRppResizeMirrorNormalize (node_resize_mirror_normalize.cpp:90-92).
 * mirror, mean, stddev may be NULL (=> no flip / no normalisation). mean/stddev are [N*C];
 * the kernel computes fmaf(v, 1/std, -(mean*(1/std))). */
RMX_API int rmx_create_resize(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                              int interpolation, int roi_type, uint32_t flags, rmx_op **out);
RMX_API int rmx_update_resize(rmx_op *op, const uint32_t *src_roi /*[N][4]*/, const uint32_t *dst_w /*[N]*/,
                              const uint32_t *dst_h /*[N]*/, const uint32_t *mirror, const float *mean,
                              const float *stddev);
/* Fused chain resize -> CropMirrorNormalize (the RandomResizedCrop + CMN graph): the resize
 * target is (dst_w,dst_h); the CMN crop window crop_roi[N][4] (x,y,w,h inside the resized image,
 * NULL = whole image) selects what is written; scale/bias as in CropMirrorNormalize. */
RMX_API int rmx_update_resize_cmn(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w,
                                  const uint32_t *dst_h, const uint32_t *crop_roi, const float *scale,
                                  const float *bias, const uint32_t *mirror);

/* Fused chain resize -> colour node -> CropMirrorNormalize for an op created with RMX_F_COLOR_LINEAR or RMX_F_COLOR_TWIST
 * (the graph rocalCropResize / rocalResize -> rocalBrightness | rocalContrast | rocalColorTwist | rocalHue | rocalSaturation
 * -> rocalCropMirrorNormalize, rocal_api_augmentation.h:67,125,237,302,794,826,878,925). c0..c3 are [N] arrays of the colour
 * node's parameters as the flag's comment lists them; a NULL array takes the neutral value (1, 0, 0, 1). The other
 * arguments are those of rmx_update_resize_cmn. */
RMX_API int rmx_update_resize_color_cmn(rmx_op *op, const uint32_t *src_roi, const uint32_t *dst_w, const uint32_t *dst_h,
                                        const uint32_t *crop_roi, const float *scale, const float *bias, const uint32_t *mirror,
                                        const float *c0, const float *c1, const float *c2, const float *c3);

/* ---- The fused chain resize -> CropMirrorNormalize in ONE call that allocates nothing. It has no counterpart in the
 *      reference; it is for callers that cannot allocate: code under HIP stream capture, tight serving loops, harnesses that
 *      forbid hipMalloc. Same arguments, kernels and results as rmx_create_resize + rmx_update_resize_cmn + rmx_op_launch
 *      (padded source tensor, no colour node in the chain: flags may hold RMX_F_QUANTIZE_U8 and RMX_F_EDGE_REF). The
 *      per-batch parameter table lives in a static device array of RMX_NOALLOC_MAX_SAMPLES rows (64 KiB on every GPU the
 *      library runs on, held until the process ends) and is written by small kernels that carry the rows as arguments, so
 *      the call makes no hipMalloc / hipFree / hipHostMalloc and no memory copy. A batch of more samples is refused.
 *      All calls on one GPU share that array: calls that overlap (two streams, two threads) race; calls on one stream
 *      are ordered by it. Asynchronous on the context's stream. ---- */
#define RMX_NOALLOC_MAX_SAMPLES 512
RMX_API int rmx_resize_cmn_noalloc(rmx_ctx *ctx, const rmx_tensor_desc *src_desc, const rmx_tensor_desc *dst_desc, int interpolation,
                                   int roi_type, uint32_t flags, const void *src, void *dst, const uint32_t *src_roi /*[N][4]*/,
                                   const uint32_t *dst_w /*[N]*/, const uint32_t *dst_h /*[N]*/, const uint32_t *crop_roi /*[N][4] or NULL*/,
                                   const float *scale /*[N*C]*/, const float *bias /*[N*C]*/, const uint32_t *mirror /*[N] or NULL*/);

/* ---- Colour family (u8 NHWC -> u8 NHWC): replaces vxExtRppColorTwist (node_color_twist.cpp:48-49),
 *      vxExtRppBrightness (node_brightness.cpp:44), vxExtRppContrast (node_contrast.cpp:44),
 *      vxExtRppHue (node_hue.cpp:42), vxExtRppSaturation (node_saturation.cpp:42). ---- */
RMX_API int rmx_create_color_twist(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                   int roi_type, rmx_op **out);
RMX_API int rmx_update_color_twist(rmx_op *op, const uint32_t *src_roi, const float *alpha,
                                   const float *beta, const float *hue_deg, const float *sat);
RMX_API int rmx_create_brightness(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                  int roi_type, rmx_op **out);
RMX_API int rmx_update_brightness(rmx_op *op, const uint32_t *src_roi, const float *alpha, const float *beta);
RMX_API int rmx_create_contrast(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                int roi_type, rmx_op **out);
RMX_API int rmx_update_contrast(rmx_op *op, const uint32_t *src_roi, const float *factor, const float *center);
RMX_API int rmx_create_hue(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                           int roi_type, rmx_op **out);
RMX_API int rmx_update_hue(rmx_op *op, const uint32_t *src_roi, const float *hue_deg);
RMX_API int rmx_create_saturation(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                  int roi_type, rmx_op **out);
RMX_API int rmx_update_saturation(rmx_op *op, const uint32_t *src_roi, const float *sat);

/* ---- Streaming neighbours of the colour family (u8 NHWC in, one pass). Their arithmetic lives in RPP, which the
 *      reference tree does not hold; the laws are the ones stated here.
 *      Gamma: replaces vxExtRppGammaCorrection (rocAL/source/augmentations/color_augmentations/node_gamma.cpp:42):
 *        out = lut[x], lut[v] = round-to-nearest-even, saturated powf(v/255, gamma)*255, one table per sample.
 *      Exposure: replaces vxExtRppExposure (node_exposure.cpp:42): out = x * 2^factor.
 *      ColorTemperature: replaces vxExtRppColorTemperature (node_color_temperature.cpp:42): red + adjustment,
 *        green unchanged, blue - adjustment, saturating.
 *      Blend: replaces vxExtRppBlend (node_blend.cpp:45): out = fmaf(a - b, ratio, b) = a*ratio + b*(1-ratio)
 *        (rocal_api_augmentation.h:371), a and b two source batches of one shape read through the first one's ROI;
 *        launched with rmx_op_launch2. ---- */
RMX_API int rmx_create_gamma(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                             int roi_type, rmx_op **out);
RMX_API int rmx_update_gamma(rmx_op *op, const uint32_t *src_roi, const float *gamma /*[N]*/);
RMX_API int rmx_create_exposure(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                int roi_type, rmx_op **out);
RMX_API int rmx_update_exposure(rmx_op *op, const uint32_t *src_roi, const float *factor /*[N]*/);
RMX_API int rmx_create_color_temperature(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                         int roi_type, rmx_op **out);
RMX_API int rmx_update_color_temperature(rmx_op *op, const uint32_t *src_roi, const int32_t *adjustment /*[N]*/);
RMX_API int rmx_create_blend(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                             int roi_type, rmx_op **out);
RMX_API int rmx_update_blend(rmx_op *op, const uint32_t *src_roi, const float *ratio /*[N]*/);
/* process step of a two-input node (Blend): as rmx_op_launch, with the second source batch. */
RMX_API int rmx_op_launch2(rmx_op *op, const void *src1, const void *src2, void *dst);

/* ---- Normalize: replaces vxExtRppNormalize (rocAL/source/augmentations/effects_augmentations/node_normalize.cpp:31-113) for image
 *      tensors: per sample, out = (x - mean) / stddev * scale + shift with the statistics taken over the axes of axis_mask
 *      (bit 0 height, bit 1 width, bit 2 channels): 3 = one mean / stddev per channel, 7 = one per sample; other masks are
 *      outside the hot path. mean and / or stddev NULL: computed on the device from the sample's window (exact integer moments,
 *      population standard deviation; a zero deviation gives out = shift); else n_stats (1 or 3) given values, as the node
 *      replicates its vectors. The arithmetic lives in RPP; the law is the one stated here: one fp32 FMA per value with
 *      a = scale / stddev and b = fma(-mean, a, shift). ---- */
RMX_API int rmx_create_normalize(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, int roi_type, rmx_op **out);
RMX_API int rmx_update_normalize(rmx_op *op, const uint32_t *src_roi, uint32_t axis_mask, const float *mean, const float *stddev,
                                 uint32_t n_stats, float scale, float shift);

/* ---- Transpose: replaces vxExtRppTranspose (rocAL/source/augmentations/geometry_augmentations/node_transpose.cpp:31-48) for image
 *      tensors. perm holds the three axes (0 height, 1 width, 2 channels) of the u8 [N,H,W,C] source in output order; on images the
 *      channel axis stays at the back or goes to the front (:52-53): {0,1,2} copy, {2,0,1} planes [N,C,H,W], {1,0,2} height and
 *      width swapped [N,W,H,C], {2,1,0} both [N,C,W,H]. The destination descriptor gives the padded size of the output's two
 *      image axes (for the swapping permutations h >= source w and w >= source h) and its layout must be the one the
 *      permutation produces; its dtype may differ from u8 (values are converted). ---- */
RMX_API int rmx_create_transpose(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst, const uint32_t *perm /*[3]*/,
                                 int roi_type, rmx_op **out);
RMX_API int rmx_update_transpose(rmx_op *op, const uint32_t *src_roi);

/* ---- WarpAffine: replaces vxExtRppWarpAffine (node_warp_affine.cpp:61-62). affine is [N][6] in
 *      rocAL's fill order x0,y0,x1,y1,o0,o1 (:43-48), read as M=[[x0,x1,o0],[y0,y1,o1]] mapping
 *      destination to source about the ROI / output centres. Out-of-ROI samples give 0. ---- */
RMX_API int rmx_create_warp_affine(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                                   int interpolation, int roi_type, rmx_op **out);
RMX_API int rmx_update_warp_affine(rmx_op *op, const uint32_t *src_roi, const float *affine /*[N][6]*/,
                                   const uint32_t *dst_w, const uint32_t *dst_h);

/* ---- Rotate: replaces vxExtRppRotate (node_rotate.cpp:43-44); angle in degrees, direction and
 *      centre as rocAL/source/meta_data/meta_node_rotate.cpp:53-77. ---- */
RMX_API int rmx_create_rotate(rmx_ctx *ctx, const rmx_tensor_desc *src, const rmx_tensor_desc *dst,
                              int interpolation, int roi_type, rmx_op **out);
RMX_API int rmx_update_rotate(rmx_op *op, const uint32_t *src_roi, const float *angle_deg /*[N]*/,
                              const uint32_t *dst_w, const uint32_t *dst_h);

/* ---- measurement helper: plain device-to-device streaming copy (nbytes, 16-byte multiples),
 *      used to establish the copy ceiling of the box and the scale of rocprof's byte counters. */
RMX_API int rmx_copy_bytes(rmx_ctx *ctx, const void *src, void *dst, size_t nbytes);
/* ---- measurement helper: one streaming pass of the same shape as the copy (every workgroup walks a contiguous chunk, four
 *      16-byte pieces per lane in flight, non-temporal loads and stores) in one of three modes: 0 copies src to dst,
 *      1 only reads src (dst is not written), 2 only writes dst (src is not read); groups_per_cu workgroups per compute
 *      unit (0: the library's default). Establishes what the memory system gives reads, writes and both together. */
RMX_API int rmx_stream_probe(rmx_ctx *ctx, int mode, const void *src, void *dst, size_t nbytes, int groups_per_cu);

#ifdef __cplusplus
}
#endif
#endif
