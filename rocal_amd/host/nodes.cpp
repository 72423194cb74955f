#include "nodes.h"

#include <algorithm>
#include <cmath>

namespace {

std::vector<uint32_t> as_u32(const std::vector<int> &v) { return std::vector<uint32_t>(v.begin(), v.end()); }

// Per-channel constants repeated for every sample: what the reference stores in its N*C vx_arrays.
std::vector<float> tile(const std::vector<float> &per_channel, size_t batch, unsigned channels) {
    std::vector<float> out(batch * channels);
    for (size_t i = 0; i < out.size(); i++) out[i] = per_channel[per_channel.size() == 1 ? 0 : i % channels];
    return out;
}

void require_mean_std(const std::vector<float> &mean, const std::vector<float> &std_dev, unsigned channels) {
    if (mean.empty() || std_dev.empty()) THROW("Mean or std dev array is empty")
    for (unsigned c = 0; c < std::min<size_t>(channels, std_dev.size()); c++)
        if (!std_dev[c]) THROW("Standard deviation value cannot be 0")
    if (channels == 3 && (mean.size() < 3 || std_dev.size() < 3)) THROW("Mean and std dev need one value per channel")
}

}  // namespace

/* ======================================================================= CropMirrorNormalize */

CropMirrorNormalizeNode::CropMirrorNormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _mirror(MIRROR_RANGE[0], MIRROR_RANGE[1]) {
    _crop_param = std::make_shared<RocalCropParam>(_batch_size);
}

void CropMirrorNormalizeNode::init(int crop_h, int crop_w, float anchor_x, float anchor_y, std::vector<float> &mean, std::vector<float> &std_dev,
                                   IntParam *mirror) {
    _crop_param->x1 = 0;
    _crop_param->y1 = 0;
    _crop_param->crop_h = crop_h;
    _crop_param->crop_w = crop_w;
    _crop_param->set_fixed_crop(anchor_x, anchor_y);
    _mean = mean;
    _std_dev = std_dev;
    _mirror.set_param(core(mirror));
}

// node_crop_mirror_normalize.cpp:56-61: scale = 1/std, bias = -(mean * scale), both in fp32.
void CropMirrorNormalizeNode::scale_bias(std::vector<float> &scale, std::vector<float> &bias) const {
    const unsigned c = _inputs[0]->info().get_channels();
    require_mean_std(_mean, _std_dev, c);
    std::vector<float> s(c), b(c);
    for (unsigned k = 0; k < c; k++) {
        const unsigned j = c == 3 ? k : 0;
        s[k] = 1 / _std_dev[j];
        b[k] = c == 3 ? -(_mean[j] * s[k]) : -(_mean[0] / _std_dev[0]);
    }
    scale = tile(s, _batch_size, c);
    bias = tile(b, _batch_size, c);
}

void CropMirrorNormalizeNode::create_node() {
    if (_node || !_scale.empty()) return;
    if (_crop_param->crop_h == 0 || _crop_param->crop_w == 0) THROW("Uninitialized destination dimension - Invalid Crop Sizes")
    _crop_param->create_array();
    scale_bias(_scale, _bias);
    _mirror.create_array(_batch_size);
    if (fused_away) return;  // the resize node in front launches the kernel for both
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_crop_mirror_normalize(_graph->get(), &s, &d, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_crop_mirror_normalize");
}

void CropMirrorNormalizeNode::refresh_for_fusion() {
    _crop_param->set_image_dimensions(_inputs[0]->info().roi());
    _crop_param->update_array();
    _outputs[0]->update_tensor_roi(_crop_param->get_cropw_arr_val(), _crop_param->get_croph_arr_val());
    _mirror.update_array();
}

void CropMirrorNormalizeNode::update_node() {
    if (fused_away) return;  // refreshed by the absorbing node, right after it has updated its output ROI
    refresh_for_fusion();
    const auto window = _crop_param->xywh();
    const auto mirror = as_u32(_mirror.values());
    check(rmx_update_crop_mirror_normalize(_node, window.data(), _scale.data(), _bias.data(), mirror.data()), "rmx_update_crop_mirror_normalize");
}

/* ======================================================================= Crop / RandomCrop / Flip */

CropNode::CropNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) : Node(inputs, outputs) {
    _crop_param = std::make_shared<RocalCropParam>(_batch_size);
}

void CropNode::init(unsigned crop_h, unsigned crop_w, float x_drift, float y_drift) {
    _crop_param->crop_w = crop_w;
    _crop_param->crop_h = crop_h;
    _crop_param->x1 = x_drift;
    _crop_param->y1 = y_drift;
    _crop_param->set_x_drift_factor(core(ParameterFactory::instance()->create_single_value_float_param(x_drift)));
    _crop_param->set_y_drift_factor(core(ParameterFactory::instance()->create_single_value_float_param(y_drift)));
}

void CropNode::init(unsigned crop_h, unsigned crop_w) {
    _crop_param->crop_w = crop_w;
    _crop_param->crop_h = crop_h;
    _crop_param->x1 = 0;
    _crop_param->y1 = 0;
    _crop_param->set_fixed_crop(0.5, 0.5);
}

void CropNode::init(FloatParam *crop_h_factor, FloatParam *crop_w_factor, FloatParam *x_drift, FloatParam *y_drift) {
    _crop_param->set_x_drift_factor(core(x_drift));
    _crop_param->set_y_drift_factor(core(y_drift));
    _crop_param->set_crop_height_factor(core(crop_h_factor));
    _crop_param->set_crop_width_factor(core(crop_w_factor));
    _crop_param->set_random();
}

void CropNode::create_node() {
    if (_node) return;
    _crop_param->create_array();
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_crop(_graph->get(), &s, &d, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_crop");
}

void CropNode::update_node() {
    _crop_param->set_image_dimensions(_inputs[0]->info().roi());
    _crop_param->update_array();
    _outputs[0]->update_tensor_roi(_crop_param->get_cropw_arr_val(), _crop_param->get_croph_arr_val());
    const auto window = _crop_param->xywh();
    check(rmx_update_crop(_node, window.data()), "rmx_update_crop");
}

RandomCropNode::RandomCropNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) : Node(inputs, outputs) {
    _crop_param = std::make_shared<RocalRandomCropParam>(_batch_size);
}

void RandomCropNode::init(FloatParam *crop_area_factor, FloatParam *crop_aspect_ratio, FloatParam *x_drift, FloatParam *y_drift, int num_of_attempts) {
    _crop_param->set_x_drift_factor(core(x_drift));
    _crop_param->set_y_drift_factor(core(y_drift));
    _crop_param->set_area_factor(core(crop_area_factor));
    _crop_param->set_aspect_ratio(core(crop_aspect_ratio));
    _num_of_attempts = num_of_attempts;  // stored and, as in the reference, not used by the window law (always 5 attempts)
}

void RandomCropNode::create_node() {
    if (_node) return;
    _crop_param->create_array();
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_crop(_graph->get(), &s, &d, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_crop");
}

void RandomCropNode::update_node() {
    _crop_param->set_image_dimensions(_inputs[0]->info().roi());
    _crop_param->update_array();
    _outputs[0]->update_tensor_roi(_crop_param->get_cropw_arr_val(), _crop_param->get_croph_arr_val());
    const auto window = _crop_param->xywh();
    check(rmx_update_crop(_node, window.data()), "rmx_update_crop");
}

FlipNode::FlipNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _horizontal(HORIZONTAL_RANGE[0], HORIZONTAL_RANGE[1]), _vertical(VERTICAL_RANGE[0], VERTICAL_RANGE[1]) {}

void FlipNode::init(int h_flag, int v_flag) {
    _horizontal.set_param(h_flag);
    _vertical.set_param(v_flag);
}

void FlipNode::init(IntParam *h_flag, IntParam *v_flag) {
    _horizontal.set_param(core(h_flag));
    _vertical.set_param(core(v_flag));
}

void FlipNode::create_node() {
    if (_node) return;
    _horizontal.create_array(_batch_size);
    _vertical.create_array(_batch_size);
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_flip(_graph->get(), &s, &d, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_flip");
}

void FlipNode::update_node() {
    _horizontal.update_array();
    _vertical.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    const auto h = as_u32(_horizontal.values()), v = as_u32(_vertical.values());
    check(rmx_update_flip(_node, roi.data(), h.data(), v.data()), "rmx_update_flip");
}

/* ======================================================================= resize family */

bool ResizeFamilyNode::try_absorb(Node *next) {
    auto *cmn = dynamic_cast<CropMirrorNormalizeNode *>(next);
    if (!cmn || _absorbed) return false;
    // Only the plain u8 resize nodes hand a u8 image to the next node; the pair then equals one resize
    // with the u8 rounding kept between the two stages.
    if (_outputs[0]->info().data_type() != RocalTensorDataType::UINT8) return false;
    if (dynamic_cast<ResizeNode *>(this) == nullptr && dynamic_cast<CropResizeNode *>(this) == nullptr) return false;
    _absorbed = cmn;
    return true;
}

bool ResizeFamilyNode::try_absorb_chain(Node *colour, Node *next) {
    const unsigned kind = colour->chain_colour_kind();
    if (!kind || _interpolation_type != ROCAL_LINEAR_INTERPOLATION) return false;
    // the colour node must hand a u8 NHWC image on, as the resize node does
    const TensorInfo &mid = colour->output()[0]->info();
    if (mid.data_type() != RocalTensorDataType::UINT8 || mid.layout() != RocalTensorlayout::NHWC) return false;
    if (!try_absorb(next)) return false;
    _absorbed_colour = colour;
    return true;
}

void ResizeFamilyNode::create_resize_op(int interpolation) {
    const TensorInfo &out = (_absorbed ? _absorbed->output()[0] : _outputs[0])->info();
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = out.desc();
    const uint32_t flags = (_absorbed ? RMX_F_QUANTIZE_U8 : 0) | (_absorbed_colour ? _absorbed_colour->chain_colour_kind() : 0) |
                           (_graph->edge_device_rule ? RMX_F_EDGE_REF : 0);
    check(rmx_create_resize(_graph->get(), &s, &d, interpolation, (int)RocalROIType::XYWH, flags, &_node), "rmx_create_resize");
}

void ResizeFamilyNode::update_resize_op(const std::vector<uint32_t> &window, const std::vector<uint32_t> &dst_w, const std::vector<uint32_t> &dst_h,
                                        const std::vector<int> *mirror, const std::vector<float> *mean, const std::vector<float> *std_dev) {
    if (_absorbed) {
        // The CMN stage sees this node's freshly updated output ROI, as it would in the two-node graph.
        _absorbed->refresh_for_fusion();
        const auto crop = _absorbed->get_crop_param()->xywh();
        const auto m = as_u32(_absorbed->mirror_values());
        if (_absorbed_colour) {
            const float *c[4];
            _absorbed_colour->chain_colour_refresh(c);
            check(rmx_update_resize_color_cmn(_node, window.data(), dst_w.data(), dst_h.data(), crop.data(), _absorbed->_scale.data(), _absorbed->_bias.data(),
                                              m.data(), c[0], c[1], c[2], c[3]),
                  "rmx_update_resize_color_cmn");
            return;
        }
        check(rmx_update_resize_cmn(_node, window.data(), dst_w.data(), dst_h.data(), crop.data(), _absorbed->_scale.data(), _absorbed->_bias.data(), m.data()),
              "rmx_update_resize_cmn");
        return;
    }
    std::vector<uint32_t> m;
    if (mirror) m = as_u32(*mirror);
    check(rmx_update_resize(_node, window.data(), dst_w.data(), dst_h.data(), mirror ? m.data() : nullptr, mean ? mean->data() : nullptr,
                            std_dev ? std_dev->data() : nullptr),
          "rmx_update_resize");
}

void ResizeFamilyNode::launch() {
    Tensor *in = _inputs[0], *out = _absorbed ? _absorbed->output()[0] : _outputs[0];
    if (!in->handle() || !out->handle()) THROW("tensor without a device buffer at launch")
    check(rmx_op_launch(_node, in->handle(), out->handle()), "rmx_op_launch");
}

void ResizeFamilyNode::adjust_out_roi_size(unsigned src_w, unsigned src_h, unsigned &dst_w, unsigned &dst_h, RocalResizeScalingMode mode, unsigned max_w,
                                           unsigned max_h) {
    const bool has_max = (max_w | max_h) > 0;
    auto cap = [&]() {
        if (!has_max) return;
        if (max_w) dst_w = std::min(dst_w, max_w);
        if (max_h) dst_h = std::min(dst_h, max_h);
    };
    switch (mode) {
        case ROCAL_SCALING_MODE_MIN_MAX: {  // max_w carries the min size, max_h the max size
            unsigned size = max_w;
            const float lo = static_cast<float>(std::min(src_w, src_h)), hi = static_cast<float>(std::max(src_w, src_h));
            if (hi / lo * size > max_h) size = static_cast<size_t>(round(max_h * lo / hi));
            if (src_w < src_h) {
                dst_w = size;
                dst_h = static_cast<size_t>(size * src_h / src_w);
            } else {
                dst_h = size;
                dst_w = static_cast<size_t>(size * src_w / src_h);
            }
            break;
        }
        case ROCAL_SCALING_MODE_STRETCH:
            if (!dst_w) dst_w = src_w;
            if (!dst_h) dst_h = src_h;
            cap();
            break;
        case ROCAL_SCALING_MODE_DEFAULT:
            if (!dst_w && dst_h)
                dst_w = std::lround(src_w * (static_cast<float>(dst_h) / src_h));
            else if (!dst_h && dst_w)
                dst_h = std::lround(src_h * (static_cast<float>(dst_w) / src_w));
            cap();
            break;
        default: {
            const float scale_w = static_cast<float>(dst_w) / src_w, scale_h = static_cast<float>(dst_h) / src_h;
            float scale = 1.0f;
            if (mode == ROCAL_SCALING_MODE_NOT_SMALLER)
                scale = std::max(scale_w, scale_h);
            else if (mode == ROCAL_SCALING_MODE_NOT_LARGER)
                scale = (scale_w > 0 && scale_h > 0) ? std::min(scale_w, scale_h) : (scale_w > 0 ? scale_w : scale_h);
            if (has_max) {
                if (max_w) scale = std::min(scale, static_cast<float>(max_w) / src_w);
                if (max_h) scale = std::min(scale, static_cast<float>(max_h) / src_h);
            }
            if (scale_h != scale || !dst_h) dst_h = std::lround(src_h * scale);
            if (scale_w != scale || !dst_w) dst_w = std::lround(src_w * scale);
        }
    }
}

void ResizeNode::init(unsigned dest_width, unsigned dest_height, RocalResizeScalingMode scaling_mode, const std::vector<unsigned> &max_size,
                      RocalResizeInterpolationType interpolation_type) {
    _interpolation_type = (int)interpolation_type;
    _scaling_mode = scaling_mode;
    _out_width = dest_width;
    _out_height = dest_height;
    if (max_size.size() > 0) {
        _max_width = max_size[0];
        _max_height = max_size[1];
    }
}

void ResizeNode::create_node() {
    if (_node) return;
    create_resize_op(_interpolation_type);
}

void ResizeNode::update_node() {
    const Roi2DCords *src = _inputs[0]->info().roi();
    const unsigned cap_w = (unsigned)_outputs[0]->info().max_shape()[0], cap_h = (unsigned)_outputs[0]->info().max_shape()[1];
    std::vector<uint32_t> dw(_batch_size), dh(_batch_size);
    for (size_t i = 0; i < _batch_size; i++) {
        unsigned w = _out_width, h = _out_height;
        adjust_out_roi_size(src[i].xywh.w, src[i].xywh.h, w, h, _scaling_mode, _max_width, _max_height);
        dw[i] = std::min(w, cap_w);
        dh[i] = std::min(h, cap_h);
    }
    _outputs[0]->update_tensor_roi(dw, dh);
    update_resize_op(roi_as_array(src), dw, dh, nullptr, nullptr, nullptr);
}

void CropResizeNode::init(float area, float aspect_ratio, float x_center_drift, float y_center_drift) {
    _crop_param = std::make_shared<RocalRandomCropParam>(_batch_size);
    _crop_param->set_area_factor(ParameterFactory::instance()->create_single_value_param(area));
    _crop_param->set_aspect_ratio(ParameterFactory::instance()->create_single_value_param(aspect_ratio));
    _crop_param->set_x_drift_factor(ParameterFactory::instance()->create_single_value_param(x_center_drift));
    _crop_param->set_y_drift_factor(ParameterFactory::instance()->create_single_value_param(y_center_drift));
}

void CropResizeNode::init(FloatParam *area, FloatParam *aspect_ratio, FloatParam *x_center_drift, FloatParam *y_center_drift) {
    _crop_param = std::make_shared<RocalRandomCropParam>(_batch_size);
    _crop_param->set_area_factor(core(area));
    _crop_param->set_aspect_ratio(core(aspect_ratio));
    _crop_param->set_x_drift_factor(core(x_center_drift));
    _crop_param->set_y_drift_factor(core(y_center_drift));
}

void CropResizeNode::init(unsigned crop_h, unsigned crop_w, float x_drift, float y_drift, RocalResizeInterpolationType interpolation_type) {
    _crop_fixed_param = std::make_shared<RocalCropParam>(_batch_size);
    _crop_fixed_param->crop_w = crop_w;
    _crop_fixed_param->crop_h = crop_h;
    _crop_fixed_param->x1 = x_drift;
    _crop_fixed_param->y1 = y_drift;
    _crop_fixed_param->set_x_drift_factor(core(ParameterFactory::instance()->create_single_value_float_param(x_drift)));
    _crop_fixed_param->set_y_drift_factor(core(ParameterFactory::instance()->create_single_value_float_param(y_drift)));
    _interpolation_type = static_cast<int>(interpolation_type);
    _is_random_crop = false;
}

void CropResizeNode::create_node() {
    if (_node) return;
    if (_is_random_crop ? !_crop_param : !_crop_fixed_param) THROW("CropResizeNode::init was not called")
    (_is_random_crop ? static_cast<CropParam *>(_crop_param.get()) : _crop_fixed_param.get())->create_array();
    create_resize_op(_interpolation_type);
}

void CropResizeNode::update_node() {
    CropParam *cp = _is_random_crop ? static_cast<CropParam *>(_crop_param.get()) : _crop_fixed_param.get();
    cp->set_image_dimensions(_inputs[0]->info().roi());
    cp->update_array();
    // As the reference (node_crop_resize.cpp:83-99): the output ROI is set to the crop size, capped to the
    // destination maxima; the destination size handed to the kernel is always the padded maximum (:38-39).
    _outputs[0]->update_tensor_roi(cp->get_cropw_arr_val(), cp->get_croph_arr_val());
    std::vector<uint32_t> dw(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[0]), dh(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[1]);
    update_resize_op(cp->xywh(), dw, dh, nullptr, nullptr, nullptr);
}

ResizeCropMirrorNode::ResizeCropMirrorNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : ResizeFamilyNode(inputs, outputs), _mirror(MIRROR_RANGE[0], MIRROR_RANGE[1]) {
    _crop_param = std::make_shared<RocalCropParam>(_batch_size);
}

void ResizeCropMirrorNode::init(unsigned crop_h, unsigned crop_w, IntParam *mirror, RocalResizeInterpolationType interpolation_type) {
    _crop_param->crop_w = crop_w;
    _crop_param->crop_h = crop_h;
    _crop_param->x1 = 0;
    _crop_param->y1 = 0;
    _mirror.set_param(core(mirror));
    _interpolation_type = static_cast<int>(interpolation_type);
}

void ResizeCropMirrorNode::init(FloatParam *crop_h_factor, FloatParam *crop_w_factor, IntParam *mirror, RocalResizeInterpolationType interpolation_type) {
    _crop_param->set_crop_height_factor(core(crop_h_factor));
    _crop_param->set_crop_width_factor(core(crop_w_factor));
    _crop_param->set_random();
    _mirror.set_param(core(mirror));
    _interpolation_type = static_cast<int>(interpolation_type);
}

void ResizeCropMirrorNode::create_node() {
    if (_node) return;
    if (_crop_param->crop_h == 0 || _crop_param->crop_w == 0) {
        // only the fixed form needs sizes; the factor form derives them from the ROI
    }
    _crop_param->create_array();
    _mirror.create_array(_batch_size);
    create_resize_op(_interpolation_type);
}

void ResizeCropMirrorNode::update_node() {
    _crop_param->set_image_dimensions(_inputs[0]->info().roi());
    _crop_param->update_array();
    _outputs[0]->update_tensor_roi(_crop_param->get_cropw_arr_val(), _crop_param->get_croph_arr_val());
    _mirror.update_array();
    std::vector<uint32_t> dw(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[0]), dh(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[1]);
    update_resize_op(_crop_param->xywh(), dw, dh, &_mirror.values(), nullptr, nullptr);
}

ResizeMirrorNormalizeNode::ResizeMirrorNormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : ResizeFamilyNode(inputs, outputs), _mirror(MIRROR_RANGE[0], MIRROR_RANGE[1]) {}

void ResizeMirrorNormalizeNode::init(unsigned dest_width, unsigned dest_height, RocalResizeScalingMode scaling_mode, std::vector<unsigned> max_size,
                                     RocalResizeInterpolationType interpolation_type, std::vector<float> &mean, std::vector<float> &std_dev, IntParam *mirror) {
    _interpolation_type = static_cast<int>(interpolation_type);
    _scaling_mode = scaling_mode;
    _out_width = dest_width;
    _out_height = dest_height;
    if (max_size.size() > 0) {
        _max_width = max_size[0];
        _max_height = max_size[1];
    }
    _mean = mean;
    _std_dev = std_dev;
    _mirror.set_param(core(mirror));
}

void ResizeMirrorNormalizeNode::create_node() {
    if (_node) return;
    const unsigned c = _inputs[0]->info().get_channels();
    require_mean_std(_mean, _std_dev, c);
    // node_resize_mirror_normalize.cpp:41-66: the raw mean / std values, repeated per sample.
    _mean_vec = tile(_mean, _batch_size, c);
    _std_vec = tile(_std_dev, _batch_size, c);
    _mirror.create_array(_batch_size);
    create_resize_op(_interpolation_type);
}

void ResizeMirrorNormalizeNode::update_node() {
    const Roi2DCords *src = _inputs[0]->info().roi();
    const unsigned cap_w = (unsigned)_outputs[0]->info().max_shape()[0], cap_h = (unsigned)_outputs[0]->info().max_shape()[1];
    std::vector<uint32_t> dw(_batch_size), dh(_batch_size);
    for (size_t i = 0; i < _batch_size; i++) {
        unsigned w = _out_width, h = _out_height;
        adjust_out_roi_size(src[i].xywh.w, src[i].xywh.h, w, h, _scaling_mode, _max_width, _max_height);
        dw[i] = std::min(w, cap_w);
        dh[i] = std::min(h, cap_h);
    }
    _outputs[0]->update_tensor_roi(dw, dh);
    _mirror.update_array();
    update_resize_op(roi_as_array(src), dw, dh, &_mirror.values(), &_mean_vec, &_std_vec);
}

/* ======================================================================= colour family */

#define RMX_COLOR_CREATE(fn)                                                                                          \
    if (_node) return;                                                                                                \
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();                                    \
    check(fn(_graph->get(), &s, &d, (int)_inputs[0]->info().roi_type(), &_node), #fn);

ColorTwistNode::ColorTwistNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _alpha(ALPHA_RANGE[0], ALPHA_RANGE[1]), _beta(BETA_RANGE[0], BETA_RANGE[1]), _hue(HUE_RANGE[0], HUE_RANGE[1]),
      _sat(SAT_RANGE[0], SAT_RANGE[1]) {}

void ColorTwistNode::init(float alpha, float beta, float hue, float sat) {
    _alpha.set_param(alpha);
    _beta.set_param(beta);
    _hue.set_param(hue);
    _sat.set_param(sat);
}

void ColorTwistNode::init(FloatParam *alpha, FloatParam *beta, FloatParam *hue, FloatParam *sat) {
    _alpha.set_param(core(alpha));
    _beta.set_param(core(beta));
    _hue.set_param(core(hue));
    _sat.set_param(core(sat));
}

void ColorTwistNode::create_node() {
    for (auto *p : {&_alpha, &_beta, &_hue, &_sat}) p->create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_color_twist)
}

void ColorTwistNode::chain_colour_refresh(const float *arrays[4]) {
    for (auto *p : {&_alpha, &_beta, &_hue, &_sat}) p->update_array();
    arrays[0] = _alpha.values().data();
    arrays[1] = _beta.values().data();
    arrays[2] = _hue.values().data();
    arrays[3] = _sat.values().data();
}

void ColorTwistNode::update_node() {
    if (fused_away) return;  // renewed by the resize node that runs the chain
    for (auto *p : {&_alpha, &_beta, &_hue, &_sat}) p->update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_color_twist(_node, roi.data(), _alpha.values().data(), _beta.values().data(), _hue.values().data(), _sat.values().data()),
          "rmx_update_color_twist");
}

BrightnessNode::BrightnessNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _alpha(ALPHA_RANGE[0], ALPHA_RANGE[1]), _beta(BETA_RANGE[0], BETA_RANGE[1]) {}

void BrightnessNode::init(float alpha, float beta) {
    _alpha.set_param(alpha);
    _beta.set_param(beta);
}

void BrightnessNode::init(FloatParam *alpha, FloatParam *beta) {
    _alpha.set_param(core(alpha));
    _beta.set_param(core(beta));
}

void BrightnessNode::create_node() {
    _alpha.create_array(_batch_size);
    _beta.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_brightness)
}

void BrightnessNode::chain_colour_refresh(const float *arrays[4]) {
    _alpha.update_array();
    _beta.update_array();
    arrays[0] = _alpha.values().data();
    arrays[1] = _beta.values().data();
    arrays[2] = arrays[3] = nullptr;
}

void BrightnessNode::update_node() {
    if (fused_away) return;
    _alpha.update_array();
    _beta.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_brightness(_node, roi.data(), _alpha.values().data(), _beta.values().data()), "rmx_update_brightness");
}

ContrastNode::ContrastNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _factor(CONTRAST_FACTOR_RANGE[0], CONTRAST_FACTOR_RANGE[1]), _center(CONTRAST_CENTER_RANGE[0], CONTRAST_CENTER_RANGE[1]) {}

void ContrastNode::init(float contrast_factor, float contrast_center) {
    _factor.set_param(contrast_factor);
    _center.set_param(contrast_center);
}

void ContrastNode::init(FloatParam *contrast_factor, FloatParam *contrast_center) {
    _factor.set_param(core(contrast_factor));
    _center.set_param(core(contrast_center));
}

void ContrastNode::create_node() {
    _factor.create_array(_batch_size);
    _center.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_contrast)
}

void ContrastNode::chain_colour_refresh(const float *arrays[4]) {  // fma(x - centre, factor, centre)
    _factor.update_array();
    _center.update_array();
    arrays[0] = _factor.values().data();
    arrays[1] = arrays[2] = _center.values().data();
    arrays[3] = nullptr;
}

void ContrastNode::update_node() {
    if (fused_away) return;
    _factor.update_array();
    _center.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_contrast(_node, roi.data(), _factor.values().data(), _center.values().data()), "rmx_update_contrast");
}

HueNode::HueNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) : Node(inputs, outputs), _hue(HUE_RANGE[0], HUE_RANGE[1]) {}
void HueNode::init(float hue) { _hue.set_param(hue); }
void HueNode::init(FloatParam *hue) { _hue.set_param(core(hue)); }

void HueNode::create_node() {
    _hue.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_hue)
}

void HueNode::chain_colour_refresh(const float *arrays[4]) {
    _hue.update_array();
    arrays[0] = arrays[1] = arrays[3] = nullptr;
    arrays[2] = _hue.values().data();
}

void HueNode::update_node() {
    if (fused_away) return;
    _hue.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_hue(_node, roi.data(), _hue.values().data()), "rmx_update_hue");
}

SaturationNode::SaturationNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _sat(SAT_RANGE[0], SAT_RANGE[1]) {}
void SaturationNode::init(float sat) { _sat.set_param(sat); }
void SaturationNode::init(FloatParam *sat) { _sat.set_param(core(sat)); }

void SaturationNode::create_node() {
    _sat.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_saturation)
}

void SaturationNode::chain_colour_refresh(const float *arrays[4]) {
    _sat.update_array();
    arrays[0] = arrays[1] = arrays[2] = nullptr;
    arrays[3] = _sat.values().data();
}

void SaturationNode::update_node() {
    if (fused_away) return;
    _sat.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_saturation(_node, roi.data(), _sat.values().data()), "rmx_update_saturation");
}

/* ======================================================================= gamma / exposure / colour temperature / blend */

GammaNode::GammaNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _gamma(GAMMA_RANGE[0], GAMMA_RANGE[1]) {}
void GammaNode::init(float gamma) { _gamma.set_param(gamma); }
void GammaNode::init(FloatParam *gamma) { _gamma.set_param(core(gamma)); }

void GammaNode::create_node() {
    _gamma.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_gamma)
}

void GammaNode::update_node() {
    _gamma.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_gamma(_node, roi.data(), _gamma.values().data()), "rmx_update_gamma");
}

NormalizeNode::NormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) : Node(inputs, outputs) {}

void NormalizeNode::init(std::vector<unsigned> &axes, std::vector<float> &mean, std::vector<float> &std_dev, float scale, float shift) {
    _mean = mean;
    _std_dev = std_dev;
    _scale = scale;
    _shift = shift;
    for (unsigned d = 0; d < axes.size(); d++) _axis_mask |= (1 << axes[d]);
}

void NormalizeNode::create_node() {
    if (_mean.size() && _std_dev.size() && _mean.size() != _std_dev.size()) THROW("Normalize: mean and stddev must hold the same number of values")
    for (float v : _std_dev)
        if (v == 0.0f) THROW("Normalize: standard deviation value cannot be 0")
    RMX_COLOR_CREATE(rmx_create_normalize)
}

void NormalizeNode::update_node() {
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    const unsigned n_stats = (unsigned)(_mean.size() ? _mean.size() : _std_dev.size());
    check(rmx_update_normalize(_node, roi.data(), (uint32_t)_axis_mask, _mean.size() ? _mean.data() : nullptr, _std_dev.size() ? _std_dev.data() : nullptr,
                               n_stats, _scale, _shift),
          "rmx_update_normalize");
}

TransposeNode::TransposeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) : Node(inputs, outputs) {}
void TransposeNode::init(std::vector<unsigned> perm) { _perm = perm; }

void TransposeNode::create_node() {
    if (_node) return;
    if (_perm.size() != 3) THROW("Transpose permutation must match with the input dims")
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_transpose(_graph->get(), &s, &d, _perm.data(), (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_transpose");
}

// node_transpose.cpp:50-66: the output ROI swaps width and height when the permutation does
void TransposeNode::update_node() {
    const Roi2DCords *src = _inputs[0]->info().roi();
    const bool swap = (_perm == std::vector<unsigned>{2, 1, 0}) || (_perm == std::vector<unsigned>{1, 0, 2});
    std::vector<uint32_t> w(_batch_size), h(_batch_size);
    for (size_t i = 0; i < _batch_size; i++) {
        w[i] = swap ? src[i].xywh.h : src[i].xywh.w;
        h[i] = swap ? src[i].xywh.w : src[i].xywh.h;
    }
    _outputs[0]->update_tensor_roi(w, h);
    const auto roi = roi_as_array(src);
    check(rmx_update_transpose(_node, roi.data()), "rmx_update_transpose");
}

ExposureNode::ExposureNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _exposure_factor(EXPOSURE_FACTOR_RANGE[0], EXPOSURE_FACTOR_RANGE[1]) {}
void ExposureNode::init(float exposure_factor) { _exposure_factor.set_param(exposure_factor); }
void ExposureNode::init(FloatParam *exposure_factor) { _exposure_factor.set_param(core(exposure_factor)); }

void ExposureNode::create_node() {
    _exposure_factor.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_exposure)
}

void ExposureNode::chain_colour_refresh(const float *arrays[4]) {  // x * 2^factor = fma(x - 0, 2^factor, 0)
    _exposure_factor.update_array();
    _multiplier.resize(_batch_size);
    for (size_t i = 0; i < _batch_size; i++) _multiplier[i] = exp2f(_exposure_factor.values()[i]);
    arrays[0] = _multiplier.data();
    arrays[1] = arrays[2] = arrays[3] = nullptr;
}

void ExposureNode::update_node() {
    if (fused_away) return;
    _exposure_factor.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_exposure(_node, roi.data(), _exposure_factor.values().data()), "rmx_update_exposure");
}

ColorTemperatureNode::ColorTemperatureNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _adj_value_param(ADJUSTMENT_RANGE[0], ADJUSTMENT_RANGE[1]) {}
void ColorTemperatureNode::init(int adjustment) { _adj_value_param.set_param(adjustment); }
void ColorTemperatureNode::init(IntParam *adjustment) { _adj_value_param.set_param(core(adjustment)); }

void ColorTemperatureNode::create_node() {
    _adj_value_param.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_color_temperature)
}

void ColorTemperatureNode::update_node() {
    _adj_value_param.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    static_assert(sizeof(int) == sizeof(int32_t), "the adjustment array is handed over as int32");
    check(rmx_update_color_temperature(_node, roi.data(), reinterpret_cast<const int32_t *>(_adj_value_param.values().data())),
          "rmx_update_color_temperature");
}

BlendNode::BlendNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _ratio(RATIO_RANGE[0], RATIO_RANGE[1]) {}
void BlendNode::init(float ratio) { _ratio.set_param(ratio); }
void BlendNode::init(FloatParam *ratio) { _ratio.set_param(core(ratio)); }

void BlendNode::create_node() {
    if (_node) return;
    if (_inputs.size() < 2) THROW("Blend node needs two input images")
    // the kernel addresses both batches with one sample stride and one row stride
    const rmx_tensor_desc a = _inputs[0]->info().desc(), b = _inputs[1]->info().desc();
    if (a.n != b.n || a.h != b.h || a.w != b.w || a.c != b.c || a.layout != b.layout || a.dtype != b.dtype)
        THROW("Blend node needs two inputs of the same shape, layout and data type")
    _ratio.create_array(_batch_size);
    RMX_COLOR_CREATE(rmx_create_blend)
}

void BlendNode::update_node() {
    _ratio.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    check(rmx_update_blend(_node, roi.data(), _ratio.values().data()), "rmx_update_blend");
}

void BlendNode::launch() {
    Tensor *in1 = _inputs[0], *in2 = _inputs[1], *out = _outputs[0];
    if (!in1->handle() || !in2->handle() || !out->handle()) THROW("tensor without a device buffer at launch")
    check(rmx_op_launch2(_node, in1->handle(), in2->handle(), out->handle()), "rmx_op_launch2");
}

/* ======================================================================= warp affine / rotate */

WarpAffineNode::WarpAffineNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _x0(COEFFICIENT_RANGE_1[0], COEFFICIENT_RANGE_1[1]), _x1(COEFFICIENT_RANGE_0[0], COEFFICIENT_RANGE_0[1]),
      _y0(COEFFICIENT_RANGE_0[0], COEFFICIENT_RANGE_0[1]), _y1(COEFFICIENT_RANGE_1[0], COEFFICIENT_RANGE_1[1]),
      _o0(COEFFICIENT_RANGE_OFFSET[0], COEFFICIENT_RANGE_OFFSET[1]), _o1(COEFFICIENT_RANGE_OFFSET[0], COEFFICIENT_RANGE_OFFSET[1]) {}

void WarpAffineNode::init(float x0, float x1, float y0, float y1, float o0, float o1, RocalResizeInterpolationType interpolation_type) {
    _x0.set_param(x0);
    _x1.set_param(x1);
    _y0.set_param(y0);
    _y1.set_param(y1);
    _o0.set_param(o0);
    _o1.set_param(o1);
    _interpolation_type = (int)interpolation_type;
}

void WarpAffineNode::init(FloatParam *x0, FloatParam *x1, FloatParam *y0, FloatParam *y1, FloatParam *o0, FloatParam *o1,
                          RocalResizeInterpolationType interpolation_type) {
    _x0.set_param(core(x0));
    _x1.set_param(core(x1));
    _y0.set_param(core(y0));
    _y1.set_param(core(y1));
    _o0.set_param(core(o0));
    _o1.set_param(core(o1));
    _interpolation_type = (int)interpolation_type;
}

// node_warp_affine.cpp:43-48,69-74: six renewals per sample, stored in the order x0,y0,x1,y1,o0,o1.
void WarpAffineNode::draw_affine() {
    _affine.resize(6 * _batch_size);
    for (size_t i = 0; i < _batch_size; i++) {
        _affine[i * 6 + 0] = _x0.renew();
        _affine[i * 6 + 1] = _y0.renew();
        _affine[i * 6 + 2] = _x1.renew();
        _affine[i * 6 + 3] = _y1.renew();
        _affine[i * 6 + 4] = _o0.renew();
        _affine[i * 6 + 5] = _o1.renew();
    }
}

void WarpAffineNode::create_node() {
    if (_node) return;
    draw_affine();
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_warp_affine(_graph->get(), &s, &d, _interpolation_type, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_warp_affine");
}

void WarpAffineNode::update_node() {
    draw_affine();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    std::vector<uint32_t> dw(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[0]), dh(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[1]);
    check(rmx_update_warp_affine(_node, roi.data(), _affine.data(), dw.data(), dh.data()), "rmx_update_warp_affine");
}

RotateNode::RotateNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
    : Node(inputs, outputs), _angle(ROTATE_ANGLE_RANGE[0], ROTATE_ANGLE_RANGE[1]) {}

void RotateNode::init(float angle, RocalResizeInterpolationType interpolation_type) {
    _angle.set_param(angle);
    _interpolation_type = (int)interpolation_type;
}

void RotateNode::init(FloatParam *angle, RocalResizeInterpolationType interpolation_type) {
    _angle.set_param(core(angle));
    _interpolation_type = (int)interpolation_type;
}

void RotateNode::create_node() {
    if (_node) return;
    _angle.create_array(_batch_size);
    rmx_tensor_desc s = _inputs[0]->info().desc(), d = _outputs[0]->info().desc();
    check(rmx_create_rotate(_graph->get(), &s, &d, _interpolation_type, (int)_inputs[0]->info().roi_type(), &_node), "rmx_create_rotate");
}

void RotateNode::update_node() {
    _angle.update_array();
    const auto roi = roi_as_array(_inputs[0]->info().roi());
    std::vector<uint32_t> dw(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[0]), dh(_batch_size, (uint32_t)_outputs[0]->info().max_shape()[1]);
    check(rmx_update_rotate(_node, roi.data(), _angle.values().data(), dw.data(), dh.data()), "rmx_update_rotate");
}
