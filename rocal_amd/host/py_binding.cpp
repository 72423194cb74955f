// Plain-C doorway for Python (ctypes) onto the entry points that take C++ types, standing where the reference's pybind
// module stands (rocAL_pybind/rocal_pybind.cpp): vectors travel as pointer + length. Every other rocal* entry point takes
// PODs only and is called by ctypes directly.
#include <cstdio>
#include <vector>

#include "crop_params.h"
#include "rocal_api_mi355x.h"

#define PY_API extern "C" __attribute__((visibility("default")))

namespace {
std::vector<float> vec(const float *p, unsigned n) { return p ? std::vector<float>(p, p + n) : std::vector<float>(); }
}  // namespace

PY_API RocalTensor rocalpy_resize(RocalContext ctx, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, int scaling_mode,
                                  const unsigned *max_size, unsigned n_max_size, unsigned resize_shorter, unsigned resize_longer, int interpolation,
                                  int layout, int dtype) {
    std::vector<unsigned> ms(max_size, max_size + (max_size ? n_max_size : 0));
    return rocalResize(ctx, in, dest_width, dest_height, is_output, (RocalResizeScalingMode)scaling_mode, ms, resize_shorter, resize_longer,
                       (RocalResizeInterpolationType)interpolation, (RocalTensorLayout)layout, (RocalTensorOutputType)dtype);
}

PY_API RocalTensor rocalpy_resize_mirror_normalize(RocalContext ctx, RocalTensor in, unsigned dest_width, unsigned dest_height, const float *mean,
                                                   unsigned n_mean, const float *std_dev, unsigned n_std, bool is_output, int scaling_mode,
                                                   const unsigned *max_size, unsigned n_max_size, unsigned resize_shorter, unsigned resize_longer,
                                                   int interpolation, RocalIntParam mirror, int layout, int dtype) {
    std::vector<float> m = vec(mean, n_mean), s = vec(std_dev, n_std);
    std::vector<unsigned> ms(max_size, max_size + (max_size ? n_max_size : 0));
    return rocalResizeMirrorNormalize(ctx, in, dest_width, dest_height, m, s, is_output, (RocalResizeScalingMode)scaling_mode, ms, resize_shorter,
                                      resize_longer, (RocalResizeInterpolationType)interpolation, mirror, (RocalTensorLayout)layout,
                                      (RocalTensorOutputType)dtype);
}

PY_API RocalTensor rocalpy_crop_mirror_normalize(RocalContext ctx, RocalTensor in, unsigned crop_height, unsigned crop_width, float start_x,
                                                 float start_y, const float *mean, unsigned n_mean, const float *std_dev, unsigned n_std,
                                                 bool is_output, RocalIntParam mirror, int layout, int dtype) {
    std::vector<float> m = vec(mean, n_mean), s = vec(std_dev, n_std);
    return rocalCropMirrorNormalize(ctx, in, crop_height, crop_width, start_x, start_y, m, s, is_output, mirror, (RocalTensorLayout)layout,
                                    (RocalTensorOutputType)dtype);
}

PY_API RocalTensor rocalpy_normalize(RocalContext ctx, RocalTensor in, const unsigned *axes, unsigned n_axes, const float *mean, unsigned n_mean,
                                     const float *std_dev, unsigned n_std, bool is_output, float scale, float shift, int dtype) {
    std::vector<unsigned> ax(axes, axes + (axes ? n_axes : 0));
    std::vector<float> m = vec(mean, n_mean), s = vec(std_dev, n_std);
    return rocalNormalize(ctx, in, ax, m, s, is_output, scale, shift, (RocalTensorOutputType)dtype);
}

PY_API RocalTensor rocalpy_transpose(RocalContext ctx, RocalTensor in, const unsigned *perm, unsigned n_perm, bool is_output, int layout) {
    return rocalTranspose(ctx, in, std::vector<unsigned>(perm, perm + (perm ? n_perm : 0)), is_output, (RocalTensorLayout)layout);
}

PY_API int rocalpy_set_outputs(RocalContext ctx, unsigned n, RocalTensor *tensors) {
    try {
        std::vector<RocalTensor> v(tensors, tensors + n);
        rocalSetOutputs(ctx, n, v);
    } catch (...) {
        return 1;
    }
    return 0;
}

// rocalGetOutputTensors for callers without C++: waits for the batch, writes up to `cap` tensor handles, returns their number (-1: error).
PY_API int rocalpy_output_tensors(RocalContext ctx, RocalTensor *out, unsigned cap) {
    RocalTensorList l = rocalGetOutputTensors(ctx);
    if (!l) return -1;
    const unsigned n = (unsigned)l->size();
    for (unsigned i = 0; i < n && i < cap; i++) out[i] = l->at(i);
    return (int)(n < cap ? n : cap);
}

PY_API void rocalpy_timing(RocalContext ctx, unsigned long long out[5]) {
    out[4] = rocalGetParameterUpdateTime(ctx);
    const TimingInfo t = rocalGetTimingInfo(ctx);
    out[0] = t.load_time;
    out[1] = t.decode_time;
    out[2] = t.process_time;
    out[3] = t.transfer_time;
}

// Windows of the decoder-side random-resized crop for a batch of image shapes (hw = height,width pairs), from a
// master seed: what rocAL's fused decoders draw per sample (parameter_random_crop_decoder.cpp:42-112).
// Writes x,y,w,h per sample and returns 0, or -1 with the message left for rocalGetErrorMessage-style callers on stderr.
PY_API int rocalpy_random_crop_dec_windows(unsigned master_seed, unsigned n, const unsigned *hw, float aspect_lo, float aspect_hi, float area_lo,
                                           float area_hi, int num_attempts, unsigned *xywh) {
    try {
        RocalRandomCropDecParam law({aspect_lo, aspect_hi}, {area_lo, area_hi}, 0, num_attempts, (int)n);
        law.generate_seeds_from(master_seed);
        for (unsigned i = 0; i < n; i++) {
            const CropWindow w = law.generate_crop_window({hw[2 * i], hw[2 * i + 1]}, (int)i);
            xywh[4 * i + 0] = w.x;
            xywh[4 * i + 1] = w.y;
            xywh[4 * i + 2] = w.W;
            xywh[4 * i + 3] = w.H;
        }
        return 0;
    } catch (const std::exception &e) {
        fprintf(stderr, "rocalpy_random_crop_dec_windows: %s\n", e.what());
        return -1;
    }
}
