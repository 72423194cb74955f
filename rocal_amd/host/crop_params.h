// Per-sample crop windows derived from the input ROI, with rocAL's class names and laws:
//   CropParam            rocAL/include/parameters/parameter_crop.h:36-92
//   RocalCropParam       rocAL/source/parameters/parameter_rocal_crop.cpp:44-85   (fixed / anchored / factor crops)
//   RocalRandomCropParam rocAL/source/parameters/parameter_random_crop.cpp:44-100 (area + aspect-ratio crops)
//   RocalRandomCropDecParam rocAL/source/parameters/parameter_random_crop_decoder.cpp:42-112 (the decoder-side
//                        random-resized-crop law: retries, fallback, integer position, one seed per sample)
// The windows feed the crop ROI argument of rmx_update_*(); the arithmetic (truncations, nearbyintf,
// number and order of random draws) is the part that has to agree with the reference.
#pragma once
#include <cmath>
#include <cstdint>
#include <random>
#include <utility>
#include <vector>

#include "parameters.h"
#include "pipeline.h"

class CropParam {
   public:
    explicit CropParam(unsigned batch_size);
    virtual ~CropParam() = default;
    void set_image_dimensions(Roi2DCords *roi) {
        if (!roi) THROW("Empty ROI ptr passed to be set to parameter_crop")
        in_roi = roi;
    }
    void set_random() { _random = true; }
    void set_fixed_crop(float anchor_x, float anchor_y) {
        _is_fixed_crop = true;
        _random = false;
        _crop_anchor[0] = anchor_x;
        _crop_anchor[1] = anchor_y;
    }
    void set_x_drift_factor(Parameter<float> *x_drift);
    void set_y_drift_factor(Parameter<float> *y_drift);
    void create_array() { array_init(); }
    virtual void update_array() {}
    const std::vector<uint32_t> &get_x1_arr_val() const { return x1_arr_val; }
    const std::vector<uint32_t> &get_y1_arr_val() const { return y1_arr_val; }
    const std::vector<uint32_t> &get_croph_arr_val() const { return croph_arr_val; }
    const std::vector<uint32_t> &get_cropw_arr_val() const { return cropw_arr_val; }
    const std::vector<uint32_t> &get_x2_arr_val() const { return x2_arr_val; }
    const std::vector<uint32_t> &get_y2_arr_val() const { return y2_arr_val; }
    void get_crop_dimensions(std::vector<uint32_t> &crop_w_dim, std::vector<uint32_t> &crop_h_dim) const {
        crop_w_dim = cropw_arr_val;
        crop_h_dim = croph_arr_val;
    }
    // x,y,w,h per sample, the form the C ABI takes
    std::vector<uint32_t> xywh() const;

    const Roi2DCords *in_roi = nullptr;
    unsigned x1 = 0, y1 = 0;
    const unsigned batch_size;

   protected:
    static constexpr float CROP_X_DRIFT_RANGE[2] = {0.01f, 0.99f};
    static constexpr float CROP_Y_DRIFT_RANGE[2] = {0.01f, 0.99f};
    void array_init();
    Parameter<float> *x_drift_factor, *y_drift_factor;
    std::vector<uint32_t> x1_arr_val, y1_arr_val, croph_arr_val, cropw_arr_val, x2_arr_val, y2_arr_val;
    bool _random = false, _is_fixed_crop = false;
    float _crop_anchor[2] = {0.5f, 0.5f};
};

class RocalCropParam : public CropParam {
   public:
    explicit RocalCropParam(unsigned batch_size);
    unsigned crop_w = 0, crop_h = 0;
    void set_crop_height_factor(Parameter<float> *f);
    void set_crop_width_factor(Parameter<float> *f);
    void update_array() override;

   private:
    static constexpr float CROP_HEIGHT_FACTOR_RANGE[2] = {0.55f, 0.95f};
    static constexpr float CROP_WIDTH_FACTOR_RANGE[2] = {0.55f, 0.95f};
    Parameter<float> *crop_height_factor, *crop_width_factor;
};

class RocalRandomCropParam : public CropParam {
   public:
    explicit RocalRandomCropParam(unsigned batch_size);
    void set_area_factor(Parameter<float> *f);
    void set_aspect_ratio(Parameter<float> *f);
    void update_array() override;

   private:
    static constexpr float AREA_FACTOR_RANGE[2] = {0.08f, 0.99f};
    static constexpr float ASPECT_RATIO_RANGE[2] = {0.7500f, 1.333f};
    Parameter<float> *area_factor, *aspect_ratio;
};

// Window of the decoder-side random crop: x, y, then height and width (parameter_random_crop_decoder.h:29-39).
struct CropWindow {
    unsigned x = 0, y = 0, H = 1, W = 1;
    CropWindow() = default;
    CropWindow(unsigned x1, unsigned y1, unsigned h, unsigned w) : x(x1), y(y1), H(h), W(w) {}
    void set_shape(unsigned h, unsigned w) { H = h, W = w; }
};

typedef std::vector<size_t> Shape;  // {height, width}
using AspectRatioRange = std::pair<float, float>;
using AreaRange = std::pair<float, float>;

// Random-resized-crop windows as rocAL's fused decoders draw them (parameter_random_crop_decoder.h:45-71): the
// engine is re-seeded per sample from a per-batch seed list, so a sample's window depends on its slot only.
// The draws per window are: up to num_attempts pairs (area fraction, log aspect ratio), then x, then y.
class RocalRandomCropDecParam {
   public:
    explicit RocalRandomCropDecParam(AspectRatioRange aspect_ratio_range = {3.0f / 4, 4.0f / 3}, AreaRange area_range = {0.08f, 1.0f},
                                     int64_t seed = 0, int num_attempts = 10, int batch_size = 256);
    CropWindow generate_crop_window(const Shape &shape, int instance);
    // Renews the factory's master seed from the random device and expands it (parameter_random_crop_decoder.cpp:108-112).
    void generate_random_seeds();
    // The same expansion from a given master seed: reproducible batches.
    void generate_seeds_from(unsigned master_seed);
    const std::vector<int> &seeds() const { return _seeds; }

   private:
    CropWindow window_for(const Shape &shape, std::mt19937 &gen);
    AspectRatioRange _aspect_ratio_range;
    std::uniform_real_distribution<float> _aspect_ratio_log_dis, _area_dis;
    std::vector<int> _seeds;
    int _num_attempts, _batch_size;
};
