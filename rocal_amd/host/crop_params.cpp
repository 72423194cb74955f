#include "crop_params.h"

#include <algorithm>
#include <mutex>

static Parameter<float> *uniform_default(const float range[2]) {
    return ParameterFactory::instance()->create_uniform_float_rand_param(range[0], range[1])->core;
}

static void replace_param(Parameter<float> *&slot, Parameter<float> *p) {
    if (!p) return;
    ParameterFactory::instance()->destroy_param(slot);
    slot = p;
}

CropParam::CropParam(unsigned n) : batch_size(n) {
    x_drift_factor = uniform_default(CROP_X_DRIFT_RANGE);
    y_drift_factor = uniform_default(CROP_Y_DRIFT_RANGE);
    array_init();
}

void CropParam::array_init() {
    for (auto *v : {&x1_arr_val, &y1_arr_val, &croph_arr_val, &cropw_arr_val, &x2_arr_val, &y2_arr_val}) v->resize(batch_size);
}

void CropParam::set_x_drift_factor(Parameter<float> *p) { replace_param(x_drift_factor, p); }
void CropParam::set_y_drift_factor(Parameter<float> *p) { replace_param(y_drift_factor, p); }

std::vector<uint32_t> CropParam::xywh() const {
    std::vector<uint32_t> out(4 * batch_size);
    for (unsigned i = 0; i < batch_size; i++) {
        out[4 * i + 0] = x1_arr_val[i];
        out[4 * i + 1] = y1_arr_val[i];
        out[4 * i + 2] = cropw_arr_val[i];
        out[4 * i + 3] = croph_arr_val[i];
    }
    return out;
}

RocalCropParam::RocalCropParam(unsigned n) : CropParam(n) {
    crop_height_factor = uniform_default(CROP_HEIGHT_FACTOR_RANGE);
    crop_width_factor = uniform_default(CROP_WIDTH_FACTOR_RANGE);
}

void RocalCropParam::set_crop_height_factor(Parameter<float> *p) { replace_param(crop_height_factor, p); }
void RocalCropParam::set_crop_width_factor(Parameter<float> *p) { replace_param(crop_width_factor, p); }

// parameter_rocal_crop.cpp:49-85. Three modes: user size at a user position, user size at an anchor
// (nearbyintf of anchor * slack, round-half-even), or random factors of the ROI (truncating casts;
// draw order per sample: height factor, width factor, x drift, y drift).
void RocalCropParam::update_array() {
    for (unsigned i = 0; i < batch_size; i++) {
        const uint32_t W = in_roi[i].xywh.w, H = in_roi[i].xywh.h;
        uint32_t cw, ch, px, py;
        if (!_random) {
            cw = (crop_w > 0 && crop_w <= W) ? crop_w : W;
            ch = (crop_h > 0 && crop_h <= H) ? crop_h : H;
            if (_is_fixed_crop) {
                px = static_cast<size_t>(std::nearbyintf(_crop_anchor[0] * (W - cw)));
                py = static_cast<size_t>(std::nearbyintf(_crop_anchor[1] * (H - ch)));
            } else {
                px = x1 >= W ? 0 : x1;
                py = y1 >= H ? 0 : y1;
            }
        } else {
            crop_height_factor->renew();
            const float fh = crop_height_factor->get();
            crop_width_factor->renew();
            const float fw = crop_width_factor->get();
            cw = static_cast<size_t>(fw * W);
            ch = static_cast<size_t>(fh * H);
            x_drift_factor->renew();
            y_drift_factor->renew();
            px = static_cast<size_t>(x_drift_factor->get() * (W - cw));
            py = static_cast<size_t>(y_drift_factor->get() * (H - ch));
        }
        x1_arr_val[i] = px;
        y1_arr_val[i] = py;
        cropw_arr_val[i] = cw;
        croph_arr_val[i] = ch;
        x2_arr_val[i] = std::min(px + cw, W);
        y2_arr_val[i] = std::min(py + ch, H);
    }
}

RocalRandomCropParam::RocalRandomCropParam(unsigned n) : CropParam(n) {
    area_factor = uniform_default(AREA_FACTOR_RANGE);
    aspect_ratio = uniform_default(ASPECT_RATIO_RANGE);
}

void RocalRandomCropParam::set_area_factor(Parameter<float> *p) { replace_param(area_factor, p); }
void RocalRandomCropParam::set_aspect_ratio(Parameter<float> *p) { replace_param(aspect_ratio, p); }

// parameter_random_crop.cpp:44-100. Up to 5 attempts of (area, aspect ratio); a candidate is kept when it
// is strictly smaller than the ROI in both directions. Sizes are truncated square roots computed in
// double from a float area factor; the y drift parameter is renewed twice per accepted attempt.
// `draw(k)` renews parameter k (0 area, 1 aspect ratio, 2 x drift, 3 y drift) and returns its value.
template <typename Draw>
static void random_crop_windows(unsigned batch_size, const Roi2DCords *in_roi, const float (&ratio_range)[2], Draw draw, std::vector<uint32_t> &x1_arr_val,
                                std::vector<uint32_t> &y1_arr_val, std::vector<uint32_t> &cropw_arr_val, std::vector<uint32_t> &croph_arr_val,
                                std::vector<uint32_t> &x2_arr_val, std::vector<uint32_t> &y2_arr_val) {
    constexpr int attempts = 5;
    for (unsigned i = 0; i < batch_size; i++) {
        const uint32_t W = in_roi[i].xywh.w, H = in_roi[i].xywh.h;
        auto fits = [&](uint32_t h, uint32_t w) { return h < H && w < W; };
        uint32_t cw = cropw_arr_val[i], ch = croph_arr_val[i];  // the last batch's values when no attempt is made
        for (int a = 0; a < attempts; a++) {
            const float area = draw(0);
            const float ratio = draw(1);
            const double target = area * H * W;  // float products, widened on assignment
            cw = static_cast<size_t>(std::sqrt(target * ratio));
            ch = static_cast<size_t>(std::sqrt(target * (1 / ratio)));
            if (fits(ch, cw)) {
                const float xd = draw(2);
                draw(3);
                const float yd = draw(3);
                x1_arr_val[i] = static_cast<size_t>(xd * (W - cw));
                y1_arr_val[i] = static_cast<size_t>(yd * (H - ch));
                break;
            }
        }
        if (!fits(ch, cw)) {  // centre crop with the aspect ratio clamped into the allowed range
            const float in_ratio = static_cast<float>(W) / H;
            if (in_ratio < ratio_range[0]) {
                cw = W;
                ch = cw / ratio_range[0];
            } else if (in_ratio > ratio_range[1]) {
                ch = H;
                cw = ch * ratio_range[1];
            } else {
                ch = H;
                cw = W;
            }
            x1_arr_val[i] = (W - cw) / 2;
            y1_arr_val[i] = (H - ch) / 2;
        }
        cropw_arr_val[i] = cw;
        croph_arr_val[i] = ch;
        x2_arr_val[i] = x1_arr_val[i] + cw;
        y2_arr_val[i] = y1_arr_val[i] + ch;
    }
}

void RocalRandomCropParam::update_array() {
    Parameter<float> *p[4] = {area_factor, aspect_ratio, x_drift_factor, y_drift_factor};
    // The usual case, four different uniform generators none of which carries an array: their locks are taken once for
    // the batch instead of once per draw (about a thousand per batch), and the draws are direct calls. Same engines, same
    // draws in the same order, same values (30.7 -> 14 us per batch of 256 together with -O3).
    UniformRand<float> *u[4];
    bool direct = true;
    for (int k = 0; k < 4; k++) {
        u[k] = dynamic_cast<UniformRand<float> *>(p[k]);
        direct = direct && u[k] != nullptr;
        for (int j = 0; j < k; j++) direct = direct && p[j] != p[k];
    }
    if (direct) {
        std::scoped_lock lock(u[0]->mutex(), u[1]->mutex(), u[2]->mutex(), u[3]->mutex());
        if (!u[0]->has_array() && !u[1]->has_array() && !u[2]->has_array() && !u[3]->has_array()) {
            random_crop_windows(batch_size, in_roi, ASPECT_RATIO_RANGE, [&](int k) { return u[k]->renew_value_unlocked(); }, x1_arr_val, y1_arr_val,
                                cropw_arr_val, croph_arr_val, x2_arr_val, y2_arr_val);
            return;
        }
    }
    random_crop_windows(batch_size, in_roi, ASPECT_RATIO_RANGE, [&](int k) {
        p[k]->renew();
        return p[k]->get();
    }, x1_arr_val, y1_arr_val, cropw_arr_val, croph_arr_val, x2_arr_val, y2_arr_val);
}

// ---- decoder-side random crop ----

RocalRandomCropDecParam::RocalRandomCropDecParam(AspectRatioRange aspect, AreaRange area, int64_t /*seed: unused by rocAL too*/, int num_attempts,
                                                 int batch_size)
    : _aspect_ratio_range(aspect),
      _aspect_ratio_log_dis(std::log(aspect.first), std::log(aspect.second)),
      _area_dis(area.first, area.second),
      _seeds(batch_size),
      _num_attempts(num_attempts),
      _batch_size(batch_size) {}

// parameter_random_crop_decoder.cpp:42-100. Kept from the reference because they decide the result: integer
// products compared against a float area, float->int truncation of the side limits, roundf of the square roots,
// the ratio test on the ROUNDED sides, the fallback that shrinks both sides by sqrt(scale) one after the other
// (the second product sees the already shrunk width), and both position draws even when their range is a single value.
CropWindow RocalRandomCropDecParam::window_for(const Shape &shape, std::mt19937 &gen) {
    if (shape.size() != 2) THROW("RocalRandomCropDecParam: shape must be {height, width}")
    CropWindow crop;
    const int H = (int)shape[0], W = (int)shape[1];
    if (W <= 0 || H <= 0) return crop;
    const float min_wh = _aspect_ratio_range.first, max_wh = _aspect_ratio_range.second;
    const float max_hw = 1 / _aspect_ratio_range.first;
    const float min_area = W * H * _area_dis.a();
    const int max_w = std::max<int>(1, H * max_wh);
    const int max_h = std::max<int>(1, W * max_hw);
    if (H * max_w < min_area) {  // too wide for any window of the smallest area
        crop.set_shape(H, max_w);
    } else if (W * max_h < min_area) {  // too tall
        crop.set_shape(max_h, W);
    } else {
        int left = _num_attempts;
        for (; left > 0; left--) {
            const float scale = _area_dis(gen);
            const size_t whole = (size_t)(H * W);
            const float target = scale * whole;
            float ratio = std::exp(_aspect_ratio_log_dis(gen));
            const int w = std::max(1, (int)std::roundf(sqrtf(target * ratio)));
            const int h = std::max(1, (int)std::roundf(sqrtf(target / ratio)));
            crop.set_shape(h, w);
            ratio = (float)w / h;
            if (w <= W && h <= H && ratio >= min_wh && ratio <= max_wh) break;
        }
        if (left <= 0) {
            const float max_area = _area_dis.b() * W * H;
            const float ratio = (float)W / H;
            if (ratio > max_wh)
                crop.set_shape(H, max_w);
            else if (ratio < min_wh)
                crop.set_shape(max_h, W);
            else
                crop.set_shape(H, W);
            const float scale = std::min(1.0f, max_area / (crop.W * crop.H));
            crop.W = std::max<int>(1, crop.W * std::sqrt(scale));
            crop.H = std::max<int>(1, crop.H * std::sqrt(scale));
        }
    }
    crop.x = std::uniform_int_distribution<int>(0, W - crop.W)(gen);
    crop.y = std::uniform_int_distribution<int>(0, H - crop.H)(gen);
    return crop;
}

CropWindow RocalRandomCropDecParam::generate_crop_window(const Shape &shape, int instance) {
    if (instance < 0 || instance >= _batch_size) THROW("RocalRandomCropDecParam: instance outside the batch")
    // one engine per thread, re-seeded per sample (parameter_random_crop_decoder.cpp:103-106)
    static thread_local std::mt19937 gen;
    gen.seed(_seeds[instance]);
    return window_for(shape, gen);
}

void RocalRandomCropDecParam::generate_random_seeds() {
    ParameterFactory::instance()->generate_seed();
    generate_seeds_from(ParameterFactory::instance()->get_seed());
}

void RocalRandomCropDecParam::generate_seeds_from(unsigned master_seed) {
    std::seed_seq seq{master_seed};
    seq.generate(_seeds.begin(), _seeds.end());
}
