// The augmentation nodes of the hot path with rocAL's class names, init() overloads and default ranges.
// create_node() builds one rmx_op where the reference calls vxExtRpp<Op>(); update_node() refreshes
// the per-sample arrays every batch where the reference refreshes its vx_arrays and crop tensor.
#pragma once
#include <memory>
#include <vector>

#include "crop_params.h"
#include "parameters.h"
#include "pipeline.h"
#include "rocal_api_mi355x.h"  // RocalResizeScalingMode, RocalResizeInterpolationType

// node_crop_mirror_normalize.cpp:34-123
class CropMirrorNormalizeNode : public Node {
   public:
    CropMirrorNormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(int crop_h, int crop_w, float anchor_x, float anchor_y, std::vector<float> &mean, std::vector<float> &std_dev, IntParam *mirror);
    std::shared_ptr<RocalCropParam> get_crop_param() { return _crop_param; }
    // for the resize node that absorbs this one
    void scale_bias(std::vector<float> &scale, std::vector<float> &bias) const;
    void refresh_for_fusion();  // the update_node() work when this node is fused away
    const std::vector<int> &mirror_values() const { return _mirror.values(); }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::shared_ptr<RocalCropParam> _crop_param;
    std::vector<float> _mean, _std_dev, _scale, _bias;
    ParameterVX<int> _mirror;
    static constexpr int MIRROR_RANGE[2] = {0, 1};
    friend class ResizeFamilyNode;
};

// node_crop.cpp:34-132
class CropNode : public Node {
   public:
    CropNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(unsigned crop_h, unsigned crop_w, float x_drift, float y_drift);
    void init(unsigned crop_h, unsigned crop_w);  // centre crop
    void init(FloatParam *crop_h_factor, FloatParam *crop_w_factor, FloatParam *x_drift, FloatParam *y_drift);
    std::shared_ptr<RocalCropParam> get_crop_param() { return _crop_param; }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::shared_ptr<RocalCropParam> _crop_param;
};

// node_random_crop.cpp:34-79
class RandomCropNode : public Node {
   public:
    RandomCropNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(FloatParam *crop_area_factor, FloatParam *crop_aspect_ratio, FloatParam *x_drift, FloatParam *y_drift, int num_of_attempts);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::shared_ptr<RocalRandomCropParam> _crop_param;
    int _num_of_attempts = 20;
};

// node_flip.cpp:31-64
class FlipNode : public Node {
   public:
    FlipNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(int h_flag, int v_flag);
    void init(IntParam *h_flag, IntParam *v_flag);
    const std::vector<int> &horizontal_values() const { return _horizontal.values(); }
    const std::vector<int> &vertical_values() const { return _vertical.values(); }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<int> _horizontal, _vertical;
    static constexpr int HORIZONTAL_RANGE[2] = {0, 1};
    static constexpr int VERTICAL_RANGE[2] = {0, 1};
};

// Shared part of the four resize nodes: one rmx resize op, per-sample destination sizes, optional
// absorbed CropMirrorNormalize.
class ResizeFamilyNode : public Node {
   public:
    using Node::Node;
    bool try_absorb(Node *next) override;
    bool try_absorb_chain(Node *colour, Node *cmn) override;
    // the resize target (the padded output size), as the reference's metadata nodes read it
    unsigned get_dst_width() { return (unsigned)_outputs[0]->info().max_shape()[0]; }
    unsigned get_dst_height() { return (unsigned)_outputs[0]->info().max_shape()[1]; }

   protected:
    void create_resize_op(int interpolation);
    // window = source window per sample (x,y,w,h); mirror/mean/std optional
    void update_resize_op(const std::vector<uint32_t> &window, const std::vector<uint32_t> &dst_w, const std::vector<uint32_t> &dst_h,
                          const std::vector<int> *mirror, const std::vector<float> *mean, const std::vector<float> *std_dev);
    void launch() override;
    // ResizeNode::adjust_out_roi_size (node_resize.cpp:98-138), with the MIN_MAX mode of
    // ResizeMirrorNormalizeNode (node_resize_mirror_normalize.cpp:138-160)
    static void adjust_out_roi_size(unsigned src_w, unsigned src_h, unsigned &dst_w, unsigned &dst_h, RocalResizeScalingMode mode,
                                    unsigned max_w, unsigned max_h);
    int _interpolation_type = ROCAL_LINEAR_INTERPOLATION;
    CropMirrorNormalizeNode *_absorbed = nullptr;
    Node *_absorbed_colour = nullptr;  // the colour node between this node and _absorbed, when the three run as one kernel
};

// node_resize.cpp:31-138
class ResizeNode : public ResizeFamilyNode {
   public:
    using ResizeFamilyNode::ResizeFamilyNode;
    void init(unsigned dest_width, unsigned dest_height, RocalResizeScalingMode scaling_mode, const std::vector<unsigned> &max_size,
              RocalResizeInterpolationType interpolation_type);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    unsigned _out_width = 0, _out_height = 0, _max_width = 0, _max_height = 0;
    RocalResizeScalingMode _scaling_mode = ROCAL_SCALING_MODE_STRETCH;
};

// node_crop_resize.cpp:32-123 (RandomResizedCrop when the window is random)
class CropResizeNode : public ResizeFamilyNode {
   public:
    using ResizeFamilyNode::ResizeFamilyNode;
    void init(float area, float aspect_ratio, float x_center_drift, float y_center_drift);
    void init(FloatParam *area, FloatParam *aspect_ratio, FloatParam *x_center_drift, FloatParam *y_center_drift);
    void init(unsigned crop_h, unsigned crop_w, float x_drift, float y_drift, RocalResizeInterpolationType interpolation_type);
    const CropParam *get_crop_param() const { return _is_random_crop ? static_cast<const CropParam *>(_crop_param.get()) : _crop_fixed_param.get(); }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::shared_ptr<RocalRandomCropParam> _crop_param;
    std::shared_ptr<RocalCropParam> _crop_fixed_param;
    bool _is_random_crop = true;
};

// node_resize_crop_mirror.cpp:33-101
class ResizeCropMirrorNode : public ResizeFamilyNode {
   public:
    ResizeCropMirrorNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(unsigned crop_h, unsigned crop_w, IntParam *mirror, RocalResizeInterpolationType interpolation_type);
    void init(FloatParam *crop_h_factor, FloatParam *crop_w_factor, IntParam *mirror, RocalResizeInterpolationType interpolation_type);
    std::shared_ptr<RocalCropParam> get_crop_param() { return _crop_param; }
    const std::vector<int> &mirror_values() const { return _mirror.values(); }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::shared_ptr<RocalCropParam> _crop_param;
    ParameterVX<int> _mirror;
    static constexpr int MIRROR_RANGE[2] = {0, 1};
};

// node_resize_mirror_normalize.cpp:34-198
class ResizeMirrorNormalizeNode : public ResizeFamilyNode {
   public:
    ResizeMirrorNormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(unsigned dest_width, unsigned dest_height, RocalResizeScalingMode scaling_mode, std::vector<unsigned> max_size,
              RocalResizeInterpolationType interpolation_type, std::vector<float> &mean, std::vector<float> &std_dev, IntParam *mirror);
    const std::vector<int> &mirror_values() const { return _mirror.values(); }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    unsigned _out_width = 0, _out_height = 0, _max_width = 0, _max_height = 0;
    RocalResizeScalingMode _scaling_mode = ROCAL_SCALING_MODE_STRETCH;
    std::vector<float> _mean, _std_dev, _mean_vec, _std_vec;
    ParameterVX<int> _mirror;
    static constexpr int MIRROR_RANGE[2] = {0, 1};
};

// color_augmentations/node_color_twist.cpp:33-74, node_brightness.cpp, node_contrast.cpp, node_hue.cpp, node_saturation.cpp
class ColorTwistNode : public Node {
   public:
    ColorTwistNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float alpha, float beta, float hue, float sat);
    void init(FloatParam *alpha, FloatParam *beta, FloatParam *hue, FloatParam *sat);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_TWIST; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _alpha, _beta, _hue, _sat;
    static constexpr float ALPHA_RANGE[2] = {0.1f, 1.95f};
    static constexpr float BETA_RANGE[2] = {0.1f, 25.0f};
    static constexpr float HUE_RANGE[2] = {5.0f, 170.0f};
    static constexpr float SAT_RANGE[2] = {0.1f, 0.4f};
};

class BrightnessNode : public Node {
   public:
    BrightnessNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float alpha, float beta);
    void init(FloatParam *alpha, FloatParam *beta);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_LINEAR; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _alpha, _beta;
    static constexpr float ALPHA_RANGE[2] = {0.1f, 1.95f};
    static constexpr float BETA_RANGE[2] = {0.0f, 25.0f};
};

class ContrastNode : public Node {
   public:
    ContrastNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float contrast_factor, float contrast_center);
    void init(FloatParam *contrast_factor, FloatParam *contrast_center);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_LINEAR; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _factor, _center;
    static constexpr float CONTRAST_FACTOR_RANGE[2] = {0.1f, 1.95f};
    static constexpr float CONTRAST_CENTER_RANGE[2] = {60.0f, 90.0f};
};

class HueNode : public Node {
   public:
    HueNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float hue);
    void init(FloatParam *hue);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_TWIST; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _hue;
    static constexpr float HUE_RANGE[2] = {-359.0f, 359.0f};
};

class SaturationNode : public Node {
   public:
    SaturationNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float sat);
    void init(FloatParam *sat);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_TWIST; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _sat;
    static constexpr float SAT_RANGE[2] = {-0.5f, 0.5f};
};

// node_gamma.cpp:28-60 (range node_gamma.h:41)
class GammaNode : public Node {
   public:
    GammaNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float gamma);
    void init(FloatParam *gamma);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _gamma;
    static constexpr float GAMMA_RANGE[2] = {0.3f, 7.00f};
};

// effects_augmentations/node_normalize.cpp:28-123: mean / standard deviation over the axes of `axes`, given or computed (an empty
// vector = computed), then scale and shift. Image tensors: axes {0,1} (per channel) or {0,1,2} (per sample).
class NormalizeNode : public Node {
   public:
    NormalizeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(std::vector<unsigned> &axes, std::vector<float> &mean, std::vector<float> &std_dev, float scale, float shift);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    int _axis_mask = 0;
    std::vector<float> _mean, _std_dev;
    float _scale = 1.0f, _shift = 0.0f;
};

// geometry_augmentations/node_transpose.cpp:28-83: perm = the input's axes (batch axis left out) in output order
class TransposeNode : public Node {
   public:
    TransposeNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(std::vector<unsigned> perm);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    std::vector<unsigned> _perm;
};

// node_exposure.cpp:28-60 (range node_exposure.h:42)
class ExposureNode : public Node {
   public:
    ExposureNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float exposure_factor);
    void init(FloatParam *exposure_factor);
    unsigned chain_colour_kind() const override { return RMX_F_COLOR_LINEAR; }
    void chain_colour_refresh(const float *arrays[4]) override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _exposure_factor;
    std::vector<float> _multiplier;  // 2^factor per sample, for the fused chain
    static constexpr float EXPOSURE_FACTOR_RANGE[2] = {0.15f, 0.95f};
};

// node_color_temperature.cpp:28-60 (integer adjustment, range node_color_temperature.h:43)
class ColorTemperatureNode : public Node {
   public:
    ColorTemperatureNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(int adjustment);
    void init(IntParam *adjustment);

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<int> _adj_value_param;
    static constexpr int ADJUSTMENT_RANGE[2] = {-99, 99};
};

// node_blend.cpp:27-66: two inputs of one shape, the first one's ROI (range node_blend.h:42)
class BlendNode : public Node {
   public:
    BlendNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float ratio);
    void init(FloatParam *ratio);
    void launch() override;

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _ratio;
    static constexpr float RATIO_RANGE[2] = {0.1f, 0.9f};
};

// node_warp_affine.cpp:37-105
class WarpAffineNode : public Node {
   public:
    WarpAffineNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float x0, float x1, float y0, float y1, float o0, float o1, RocalResizeInterpolationType interpolation_type);
    void init(FloatParam *x0, FloatParam *x1, FloatParam *y0, FloatParam *y1, FloatParam *o0, FloatParam *o1,
              RocalResizeInterpolationType interpolation_type);
    const std::vector<float> &affine() const { return _affine; }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    void draw_affine();
    ParameterVX<float> _x0, _x1, _y0, _y1, _o0, _o1;
    std::vector<float> _affine;
    int _interpolation_type = ROCAL_LINEAR_INTERPOLATION;
    static constexpr float COEFFICIENT_RANGE_0[2] = {-0.35f, 0.35f};
    static constexpr float COEFFICIENT_RANGE_1[2] = {0.65f, 1.35f};
    static constexpr float COEFFICIENT_RANGE_OFFSET[2] = {-10.0f, 10.0f};
};

// node_rotate.cpp:30-61
class RotateNode : public Node {
   public:
    RotateNode(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs);
    void init(float angle, RocalResizeInterpolationType interpolation_type);
    void init(FloatParam *angle, RocalResizeInterpolationType interpolation_type);
    const std::vector<float> &angle_values() const { return _angle.values(); }
    unsigned get_dst_width() { return (unsigned)_outputs[0]->info().max_shape()[0]; }
    unsigned get_dst_height() { return (unsigned)_outputs[0]->info().max_shape()[1]; }

   protected:
    void create_node() override;
    void update_node() override;

   private:
    ParameterVX<float> _angle;
    int _interpolation_type = ROCAL_LINEAR_INTERPOLATION;
    static constexpr float ROTATE_ANGLE_RANGE[2] = {0.0f, 180.0f};
};
