/*
 * rocal_oracle.h - CPU restatement of rocAL's augmentation hot path (TEST INFRASTRUCTURE ONLY).
 *
 * This is the checker the HIP kernels are compared against. It is never linked into,
 * imported by, or called from the shipped library: only tests/, the smoke check and the
 * cpu_baseline leg of the benchmark may load it.
 *
 * rocAL itself holds no pixel arithmetic for these ops: every node forwards to RPP through
 * MIVisionX's vx_rpp extension (e.g. rocAL/source/augmentations/geometry_augmentations/
 * node_crop_mirror_normalize.cpp:87, node_resize.cpp:56, node_warp_affine.cpp:61,
 * color_augmentations/node_color_twist.cpp:48). RPP and MIVisionX are third-party
 * dependencies absent from the reference tree (rocAL/CMakeLists.txt:131-133 requires
 * "MIVisionX"; no version pin beyond "vx_rpp >= 3.1.0", rocAL/CMakeLists.txt:338).
 * Each function below therefore follows the in-tree text that restates the algorithm and
 * says which clauses are DEFINED here because nothing in the tree pins them.
 *
 * Pin status per function (what independent evidence each has):
 *   orc_crop_mirror_normalize  pinned: closed form (integer gather + one fp32 FMA), brute force.
 *   orc_resize (bilinear)      pinned: in-tree kernel rocAL/rocAL_hip/rocal_hip_kernels.cpp:311-485
 *                              (compiled as oracle/_ref and compared on the GPU with
 *                              ORC_F_BILINEAR_EDGE_QUIRK; that source builds `(float4)scalar` as
 *                              (scalar,0,0,0) under this toolchain's HIP headers, so the comparison
 *                              holds on lane 0 of each 8-pixel group at vertical ratio 1: x law,
 *                              weights, fmaf chain, edge clamp and the rounding store, bit-exact),
 *                              torch F.interpolate closed forms, box-mean and ramp special cases
 *                              for both axes. Which edge clamp RPP's HOST path uses (hi or hi-1)
 *                              is parity unpinned; the default is the textbook clamp to hi.
 *   orc_resize (triangular)    pinned: in-tree kernel rocal_hip_kernels.cpp:487-589 (oracle/_ref,
 *                              ORC_F_ROUND_TRUNC), partition of unity, box-mean special cases.
 *   orc_to_tensor              pinned: rocal_hip_kernels.cpp:131-217 (oracle/_ref), closed form.
 *   orc_brightness/contrast    parity unpinned beyond the closed form alpha*x+beta (API doc
 *                              rocAL/include/api/rocal_api_augmentation.h:231-232).
 *   orc_gamma/exposure/color_temperature/blend
 *                              PARITY UNPINNED against RPP; closed forms tested (gamma 1 and 2, 2^k
 *                              exposure, saturating +-adj, ratio 0 / 1 / 0.5).
 *   orc_resize (nearest)       law DEFINED here (floor of the half-pixel-centre coordinate + 0.5); the restatement is
 *                              checked against hand-written indices (identity, 2x / 3x down, 2x / 3x replication, ROI and
 *                              mirror); against RPP it is parity unpinned.
 *   orc_normalize              law DEFINED here (PARITY UNPINNED against RPP); the restatement is checked against numpy's mean / std in
 *                              float64, a constant image (out = shift) and a two-valued image with hand-computed statistics.
 *   orc_color_twist/hue/sat    restatement checked on all 2^24 RGB triples against the same HSV round trip written
 *                              with true divisions in numpy (5 parameter sets: at most one level apart, < 0.3 % of
 *                              values differ), identity, grey fixed points, 360-periodicity, colorsys. Against RPP the
 *                              HSV formulation is PARITY UNPINNED (it lives only in RPP).
 *   orc_warp_affine            restatement checked by exact dyadic blends of fractional translations (weight order,
 *                              neighbours, far-edge clamp), the out-of-ROI rule at floor == lo-1 / hi / hi+1, a float64
 *                              brute force for rotation+scale+shift with an off-origin ROI and another destination
 *                              size, and torch grid_sample in the interior. Matrix element order and centre
 *                              convention are PARITY UNPINNED against RPP.
 *   orc_rotate                 direction/centre pinned by rocAL/source/meta_data/meta_node_rotate.cpp:53-77;
 *                              fp path from angle to matrix PARITY UNPINNED.
 *   parameter laws (orc_mt19937*, orc_seed_seq, orc_uniform_rand*, orc_custom_rand,
 *   orc_fixed_crop, orc_random_crop, orc_factor_crop)
 *                              pinned: C++ standard known answers (10000th mt19937 output),
 *                              libstdc++ cross-check in tests.
 */
#ifndef ROCAL_ORACLE_H
#define ROCAL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* rocAL/include/pipeline/commons.h:45-70 */
enum { ORC_NHWC = 0, ORC_NCHW = 1 };
enum { ORC_FP32 = 0, ORC_FP16 = 1, ORC_UINT8 = 2 };
/* rocAL/include/api/rocal_api_types.h:347-366 */
enum { ORC_INTERP_NEAREST = 0, ORC_INTERP_LINEAR = 1, ORC_INTERP_TRIANGULAR = 5 };

/* convention switches (defaults = 0) */
enum {
    ORC_F_ROUND_TRUNC = 1u << 0,          /* u8 store truncates instead of round-to-nearest-even */
    ORC_F_BILINEAR_EDGE_QUIRK = 1u << 1,  /* clamp both neighbours to hi-1 (rocal_hip_kernels.cpp:340-343) */
    ORC_F_TRI_2D = 1u << 2,               /* triangular: 2-D non-separable accumulation (rocal_hip_kernels.cpp:568-586) */
    ORC_F_QUANTIZE_U8 = 1u << 3,          /* resize result rounded to u8 before normalisation (two-node rocAL graph) */
    ORC_F_FP16_TRUNC = 1u << 4,           /* fp16 store rounds toward zero (master_graph.cpp:819-821) */
    ORC_F_HUE_INT_TRUNC = 1u << 5         /* hue degrees truncated to int and taken mod 360 first */
};

/* Image batch view: u8, NHWC with C channels, sample stride = hmax*wmax*c bytes, row stride wmax*c.
 * (rocAL/source/pipeline/tensor.cpp:116-137, loaders/image/image_read_and_decode.cpp:188-195) */
typedef struct {
    const uint8_t *data;
    int n, hmax, wmax, c;
} orc_src;

/* Output batch view. dtype/layout per enums above; dims are the padded maxima. */
typedef struct {
    void *data;
    int n, hmax, wmax, c;
    int layout;
    int dtype;
} orc_dst;

uint16_t orc_f32_to_f16(float v, int trunc);
float orc_f16_to_f32(uint16_t h);

/* out[n,c,y,x] = fmaf((float)in[n, y1+y, x1+(mirror? cw-1-x : x), c], scale[n*C+c], bias[n*C+c]).
 * vflip (nullable) reverses rows (used by Flip). crop_xywh is [n][4] = x,y,w,h. */
void orc_crop_mirror_normalize(const orc_src *src, const uint32_t *crop_xywh,
                               const float *scale, const float *bias,
                               const uint32_t *mirror, const uint32_t *vflip,
                               const orc_dst *dst, unsigned flags);

/* rocAL's derivation of scale/bias from mean/std (node_crop_mirror_normalize.cpp:56-61). */
void orc_cmn_scale_bias(const float *mean, const float *stddev, int c, int n, float *scale, float *bias);

/* Resize ROI -> (dst_w[i], dst_h[i]); optional mirror (destination x reversed) and
 * normalisation (scale/bias nullable => identity and the output is the rounded u8 value cast
 * to the destination type when dtype != u8). */
void orc_resize(const orc_src *src, const uint32_t *roi_xywh,
                const uint32_t *dst_w, const uint32_t *dst_h, int interp,
                const uint32_t *mirror, const float *scale, const float *bias,
                const orc_dst *dst, unsigned flags);

/* out = fmaf(x, alpha, beta) -> u8 */
void orc_brightness(const orc_src *src, const uint32_t *roi_xywh, const float *alpha, const float *beta,
                    const orc_dst *dst, unsigned flags);
/* out = fmaf(x - center, factor, center) -> u8 */
void orc_contrast(const orc_src *src, const uint32_t *roi_xywh, const float *factor, const float *center,
                  const orc_dst *dst, unsigned flags);
/* Gamma / Exposure / ColorTemperature / Blend: laws DEFINED in rocal_oracle.c (parity unpinned against RPP). */
void orc_gamma_lut(float gamma, uint8_t *lut /*[256]*/, unsigned flags);
void orc_gamma(const orc_src *src, const uint32_t *roi_xywh, const float *gamma, const orc_dst *dst, unsigned flags);
void orc_exposure(const orc_src *src, const uint32_t *roi_xywh, const float *factor, const orc_dst *dst, unsigned flags);
void orc_color_temperature(const orc_src *src, const uint32_t *roi_xywh, const int32_t *adjustment, const orc_dst *dst,
                           unsigned flags);
/* axis_mask 3 (height, width) or 7 (height, width, channels); mean / stddev NULL = computed; n_stats 1 or 3 given values */
void orc_normalize(const orc_src *src, const uint32_t *roi_xywh, unsigned axis_mask, const float *mean, const float *stddev, unsigned n_stats,
                   float scale, float shift, const orc_dst *dst, unsigned flags);
void orc_blend(const orc_src *src1, const orc_src *src2, const uint32_t *roi_xywh, const float *ratio, const orc_dst *dst,
               unsigned flags);
/* HSV colour twist; hue in degrees. */
void orc_color_twist(const orc_src *src, const uint32_t *roi_xywh, const float *alpha, const float *beta,
                     const float *hue, const float *sat, const orc_dst *dst, unsigned flags);

/* affine is [n][6] = m0..m5 with (sx,sy) = M*(dx-dcx, dy-dcy, 1) + src centre. */
void orc_warp_affine(const orc_src *src, const uint32_t *roi_xywh, const float *affine, int interp,
                     const uint32_t *dst_w, const uint32_t *dst_h, const orc_dst *dst, unsigned flags);
/* Build the inverse-map matrix for a rotation of angle degrees. */
void orc_rotate_matrix(float angle_deg, float m[6]);
/* rocAL's six floats (x0,y0,x1,y1,o0,o1; node_warp_affine.cpp:43-48) -> m0..m5. */
void orc_affine_from_rocal(const float a[6], float m[6]);

/* Second-pass normalise/transpose of MasterGraph::to_tensor (master_graph.cpp:672-853). */
void orc_to_tensor(const uint8_t *src, int n, int h, int w, int c, const float mul[3], const float add[3],
                   int reverse_channels, const orc_dst *dst, unsigned flags);

/* ---- host-side parameter laws ---- */
typedef struct { uint32_t mt[624]; int idx; } orc_mt19937;
void orc_mt19937_seed(orc_mt19937 *g, uint32_t seed);
uint32_t orc_mt19937_next(orc_mt19937 *g);
/* std::seed_seq{seed}.generate(out, out+n) */
void orc_seed_seq_generate(const uint32_t *seeds, int nseeds, uint32_t *out, int n);
/* UniformRand<float>::renew_value (parameter_random.h:59-71) */
float orc_uniform_rand_f32(orc_mt19937 *g, float start, float end);
int orc_uniform_rand_i32(orc_mt19937 *g, int start, int end);
/* CustomRand<int>::renew_value (parameter_random.h:176-193); returns index into values */
int orc_custom_rand_index(orc_mt19937 *g, const double *freq, int size);
/* RocalCropParam::fill_crop_dims, fixed branch (parameter_rocal_crop.cpp:49-85); out = x1,y1,w,h */
void orc_fixed_crop(uint32_t roi_w, uint32_t roi_h, uint32_t crop_w, uint32_t crop_h,
                    int is_fixed_anchor, float anchor_x, float anchor_y, uint32_t x1, uint32_t y1,
                    uint32_t out_xywh[4]);
/* A float parameter as the crop laws see it: either a UniformRand<float> (own generator, one draw per
 * renew) or a SimpleParameter<float> (renew draws nothing). */
typedef struct { orc_mt19937 g; float lo, hi; int simple; float value; } orc_fparam;
void orc_fparam_uniform(orc_fparam *p, float lo, float hi, uint32_t seed); /* constructor draws once (parameter_random.h:40-43) */
void orc_fparam_simple(orc_fparam *p, float value);
float orc_fparam_renew(orc_fparam *p);
/* RocalRandomCropParam::fill_crop_dims for one sample (parameter_random_crop.cpp:44-100); out = x1,y1,w,h.
 * prev_wh = this sample's w,h from the previous batch (what the arrays still hold). */
void orc_random_crop(orc_fparam *area, orc_fparam *aspect, orc_fparam *x_drift, orc_fparam *y_drift,
                     uint32_t roi_w, uint32_t roi_h, uint32_t out_xywh[4]);
/* RocalCropParam::fill_crop_dims, random-factor branch (parameter_rocal_crop.cpp:66-78) */
void orc_factor_crop(orc_fparam *h_factor, orc_fparam *w_factor, orc_fparam *x_drift, orc_fparam *y_drift,
                     uint32_t roi_w, uint32_t roi_h, uint32_t out_xywh[4]);
/* ResizeNode::adjust_out_roi_size (node_resize.cpp:98-138). mode: 0 default,1 stretch,2 not_smaller,3 not_larger */
void orc_resize_out_size(unsigned src_w, unsigned src_h, unsigned dst_w, unsigned dst_h, int mode,
                         unsigned max_w, unsigned max_h, unsigned *out_w, unsigned *out_h);

int orc_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
