// rocAL C API entry points of the hot-path operators (rocAL/source/api/rocal_api.cpp:82-107,
// rocal_api_parameter.cpp, rocal_api_augmentation.cpp). Each one derives the output TensorInfo from the
// input's exactly as the reference does, adds the node and calls its init(); exceptions are caught here,
// stored in the context, printed, and turned into a null tensor / ROCAL_RUNTIME_ERROR.
#include "rocal_host.h"
#include "nodes.h"

#include "meta.h"

#include <iostream>
#include <type_traits>

namespace {

void report(Context *context, const std::exception &e) {
    context->capture_error(e.what());
    std::cerr << e.what() << std::endl;
}

// MasterGraph::meta_add_node (master_graph.h:265-273): the metadata twin of an augmentation node
template <typename MetaT, typename NodeT>
void meta_add_node(Context *context, std::shared_ptr<NodeT> node) {
    if (!context->master_graph->meta_data_enabled()) return;
    auto meta_node = std::make_shared<MetaT>();
    meta_node->_node = node;
    meta_node->_batch_size = (int)context->master_graph->batch_size();
    context->master_graph->meta_graph()->_meta_nodes.push_back(meta_node);
}

// which metadata node follows which augmentation node (rocal_api_augmentation.cpp: the meta_add_node calls)
template <typename NodeT> struct MetaOf { using type = void; };
template <> struct MetaOf<CropNode> { using type = CropMetaNode; };
template <> struct MetaOf<CropMirrorNormalizeNode> { using type = CropMirrorNormalizeMetaNode; };
template <> struct MetaOf<CropResizeNode> { using type = CropResizeMetaNode; };
template <> struct MetaOf<ResizeNode> { using type = ResizeMetaNode; };
template <> struct MetaOf<ResizeCropMirrorNode> { using type = ResizeCropMirrorMetaNode; };
template <> struct MetaOf<ResizeMirrorNormalizeNode> { using type = ResizeMirrorNormalizeMetaNode; };
template <> struct MetaOf<FlipNode> { using type = FlipMetaNode; };
template <> struct MetaOf<RotateNode> { using type = RotateMetaNode; };

enum class Dims { KEEP, SET };

// Common frame of every augmentation entry point.
template <typename NodeT, typename InitFn>
Tensor *add_op(RocalContext p_context, RocalTensor p_input, bool is_output, RocalTensorLayout output_layout, RocalTensorOutputType output_datatype,
               Dims dims, unsigned width, unsigned height, const char *precondition_error, InitFn init, RocalTensor p_input2 = nullptr,
               bool two_inputs = false) {
    Tensor *output = nullptr;
    if (!p_context) {
        std::cerr << "Invalid rocal context passed" << std::endl;
        return output;
    }
    auto *context = static_cast<Context *>(p_context);
    if (!p_input || (two_inputs && !p_input2)) {
        context->capture_error("Invalid rocal tensor passed");
        std::cerr << "Invalid rocal tensor passed" << std::endl;
        return output;
    }
    auto *input = static_cast<Tensor *>(p_input);
    try {
        if (precondition_error) THROW(precondition_error)
        if (context->master_graph->built()) THROW("the graph is already verified; nodes cannot be added")
        TensorInfo output_info = input->info();
        const auto layout = static_cast<RocalTensorlayout>(output_layout);
        output_info.set_data_type(static_cast<RocalTensorDataType>(output_datatype));
        if (dims == Dims::SET)
            output_info.modify_dims_width_and_height(layout, width, height);
        else
            output_info.set_tensor_layout(layout);
        output = context->master_graph->create_tensor(output_info, is_output);
        std::vector<Tensor *> inputs{input};
        if (two_inputs) inputs.push_back(static_cast<Tensor *>(p_input2));
        auto node = context->master_graph->add_node<NodeT>(inputs, {output});
        init(*node);
        if constexpr (!std::is_void<typename MetaOf<NodeT>::type>::value) meta_add_node<typename MetaOf<NodeT>::type, NodeT>(context, node);
    } catch (const std::exception &e) {
        report(context, e);
        output = nullptr;
    }
    return output;
}

FloatParam *F(RocalFloatParam p) { return static_cast<FloatParam *>(p); }
IntParam *I(RocalIntParam p) { return static_cast<IntParam *>(p); }

}  // namespace

/* ------------------------------------------------------------------ context */

RocalContext rocalCreate(size_t batch_size, RocalProcessMode affinity, int gpu_id, size_t, size_t, RocalTensorOutputType) {
    try {
        if (batch_size == 0) THROW("batch size must be positive")
        if (affinity != ROCAL_PROCESS_GPU) THROW("only ROCAL_PROCESS_GPU is available: this build has no CPU path")
        return new Context(batch_size, gpu_id, nullptr);
    } catch (const std::exception &e) {
        std::cerr << e.what() << std::endl;
        return nullptr;
    }
}

RocalStatus rocalVerify(RocalContext p_context) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->build();
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

RocalStatus rocalRun(RocalContext p_context) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->run();
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

// Loader threads blocked on a packed source are woken and turned away first (image_loader.cpp:84,126-127); the
// destructor of the graph frees the rings only when they have left.
RocalStatus rocalRelease(RocalContext p_context) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    context->master_graph->stop_sources();
    delete context;
    return ROCAL_OK;
}

RocalStatus rocalSetBilinearEdgeRule(RocalContext p_context, int device_rule) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->set_edge_rule(device_rule != 0);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

const char *rocalGetErrorMessage(RocalContext p_context) { return p_context ? static_cast<Context *>(p_context)->error.c_str() : "Invalid rocal context passed"; }

/* ------------------------------------------------------------------ decoded batches in device memory */

RocalTensor rocalDeviceSource(RocalContext p_context, unsigned max_width, unsigned max_height, bool is_output) {
    if (!p_context) return nullptr;
    auto *context = static_cast<Context *>(p_context);
    try {
        if (max_width == 0 || max_height == 0) THROW("source needs non-zero maximum dimensions")
        TensorInfo info({context->master_graph->batch_size(), max_height, max_width, 3}, RocalTensorlayout::NHWC, RocalTensorDataType::UINT8);
        return context->master_graph->create_tensor(info, is_output);
    } catch (const std::exception &e) {
        report(context, e);
        return nullptr;
    }
}

RocalStatus rocalDeviceSourceFeed(RocalContext p_context, RocalTensor p_source, const void *device_ptr, const unsigned *roi_width, const unsigned *roi_height) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        if (!p_source || !device_ptr || !roi_width || !roi_height) THROW("null argument")
        auto *t = static_cast<Tensor *>(p_source);
        const size_t n = t->info().batch_size();
        t->swap_handle(const_cast<void *>(device_ptr));
        t->update_tensor_roi(std::vector<uint32_t>(roi_width, roi_width + n), std::vector<uint32_t>(roi_height, roi_height + n));
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

/* ------------------------------------------------------------------ packed batches from a loader */

RocalTensor rocalPackedSource(RocalContext p_context, unsigned max_width, unsigned max_height, bool is_output, unsigned queue_depth, size_t slot_bytes) {
    if (!p_context) return nullptr;
    auto *context = static_cast<Context *>(p_context);
    try {
        if (max_width == 0 || max_height == 0) THROW("source needs non-zero maximum dimensions")
        const size_t n = context->master_graph->batch_size();
        TensorInfo info({n, max_height, max_width, 3}, RocalTensorlayout::NHWC, RocalTensorDataType::UINT8);
        // default capacity: every image at its maximum size (what the padded tensor of the reference takes)
        if (slot_bytes == 0) slot_bytes = n * (size_t)max_height * (((size_t)max_width * 3 + 3) / 4 * 4);
        return context->master_graph->create_packed_source(info, is_output, slot_bytes, queue_depth < 2 ? 2 : queue_depth);
    } catch (const std::exception &e) {
        report(context, e);
        return nullptr;
    }
}

unsigned char *rocalPackedSourcePlaceImage(RocalContext p_context, RocalTensor p_source, unsigned index, unsigned width, unsigned height, unsigned *row_stride) {
    if (!p_context) return nullptr;
    auto *context = static_cast<Context *>(p_context);
    try {
        auto *t = static_cast<Tensor *>(p_source);
        if (!t) THROW("null source")
        const auto &shape = t->info().max_shape();
        if (width > shape[0] || height > shape[1]) THROW("image of " + TOSTR(width) + " x " + TOSTR(height) + " exceeds the source's maximum of " + TOSTR(shape[0]) + " x " + TOSTR(shape[1]))
        return context->master_graph->packed_buffer(t)->place_image(index, width, height, row_stride);
    } catch (const std::exception &e) {
        report(context, e);
        return nullptr;
    }
}

RocalStatus rocalPackedSourcePush(RocalContext p_context, RocalTensor p_source) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->packed_buffer(static_cast<Tensor *>(p_source))->push();
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

RocalStatus rocalPackedSourceStop(RocalContext p_context, RocalTensor p_source) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->packed_buffer(static_cast<Tensor *>(p_source))->stop();
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

RocalStatus rocalPackedSourceWait(RocalContext p_context, RocalTensor p_source) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        PackedCircularBuffer *ring = context->master_graph->packed_buffer(static_cast<Tensor *>(p_source));
        ring->block_if_empty();
        if (ring->stopped()) THROW("the packed batch buffer was released")
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

size_t rocalPackedSourceLevel(RocalContext p_context, RocalTensor p_source) {
    if (!p_context) return 0;
    auto *context = static_cast<Context *>(p_context);
    try {
        return context->master_graph->packed_buffer(static_cast<Tensor *>(p_source))->level();
    } catch (const std::exception &e) {
        report(context, e);
        return 0;
    }
}

void rocalSetOutputs(RocalContext p_context, unsigned int num_of_outputs, std::vector<RocalTensor> &output_tensors) {
    if (!p_context) THROW("Invalid rocal context passed to rocalSetOutputs")
    auto *context = static_cast<Context *>(p_context);
    if (num_of_outputs > output_tensors.size()) THROW("rocalSetOutputs: fewer tensors than announced")
    for (unsigned i = 0; i < num_of_outputs; i++) context->master_graph->set_output(static_cast<Tensor *>(output_tensors[i]));
}

RocalStatus rocalTensorInfo(RocalTensor p_tensor, size_t dims[4], int *layout, int *data_type) {
    if (!p_tensor || !dims || !layout || !data_type) return ROCAL_INVALID_PARAMETER_TYPE;
    const TensorInfo &info = static_cast<Tensor *>(p_tensor)->info();
    for (size_t i = 0; i < 4; i++) dims[i] = i < info.dims().size() ? info.dims()[i] : 1;
    *layout = (int)info.layout();
    *data_type = (int)info.data_type();
    return ROCAL_OK;
}

RocalStatus rocalTensorSetBuffer(RocalContext p_context, RocalTensor p_tensor, void *device_ptr) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->bind_output(static_cast<Tensor *>(p_tensor), device_ptr);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

// rocal_api_info.cpp:90-97
TimingInfo rocalGetTimingInfo(RocalContext p_context) {
    TimingInfo info{0, 0, 0, 0};
    if (!p_context) return info;
    auto *context = static_cast<Context *>(p_context);
    unsigned long long t[3];
    context->master_graph->take_timing(t);
    context->update_time_us += t[0];
    info.process_time = t[1];
    info.transfer_time = t[2];
    return info;
}

long long unsigned rocalGetParameterUpdateTime(RocalContext p_context) {
    if (!p_context) return 0;
    auto *context = static_cast<Context *>(p_context);
    unsigned long long t[3];
    // (the other two timers are kept for the next rocalGetTimingInfo)
    context->master_graph->take_timing(t);
    context->master_graph->give_back_timing(t[1], t[2]);
    const unsigned long long r = context->update_time_us + t[0];
    context->update_time_us = 0;
    return r;
}

void *rocalTensorBuffer(RocalTensor t) {
    try {
        return t ? t->buffer() : nullptr;  // (waits for the batch that is being computed)
    } catch (const std::exception &e) {
        std::cerr << e.what() << std::endl;
        return nullptr;
    }
}
const unsigned *rocalTensorRoi(RocalTensor t) { return t ? reinterpret_cast<const unsigned *>(static_cast<Tensor *>(t)->info().roi()) : nullptr; }
size_t rocalTensorDataSize(RocalTensor t) { return t ? static_cast<Tensor *>(t)->info().data_size() : 0; }

/* ------------------------------------------------------------------ results (rocal_api_data_transfer.cpp:54-68,110-121) */

RocalTensorList rocalGetOutputTensors(RocalContext p_context) {
    if (!p_context) return nullptr;
    auto *context = static_cast<Context *>(p_context);
    try {
        return context->master_graph->get_output_tensors();
    } catch (const std::exception &e) {
        report(context, e);
        return nullptr;
    }
}

RocalStatus rocalCopyToOutput(RocalContext p_context, unsigned char *out_ptr, size_t out_size) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->copy_output(out_ptr, out_size);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

RocalStatus rocalOutputsWaitOnStream(RocalContext p_context, void *stream) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->outputs_wait_on_stream(stream);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

/* ------------------------------------------------------------------ output conversion (rocal_api_data_transfer.cpp:30-52) */

RocalStatus rocalToTensor(RocalContext p_context, void *out_ptr, RocalTensorLayout tensor_format, RocalTensorOutputType tensor_output_type,
                          float multiplier0, float multiplier1, float multiplier2, float offset0, float offset1, float offset2, bool reverse_channels,
                          RocalOutputMemType output_mem_type, int max_roi_height, int max_roi_width) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        if (tensor_format != ROCAL_NHWC && tensor_format != ROCAL_NCHW) THROW("Supported only for NHWC and NCHW tensor layout")
        if (tensor_output_type != ROCAL_FP32 && tensor_output_type != ROCAL_FP16) THROW("Supported only for FP32 and FP16 tensor data types")
        if (output_mem_type != ROCAL_MEMCPY_GPU) THROW("only ROCAL_MEMCPY_GPU is available: this build has no host path")
        if (max_roi_height < 0 || max_roi_width < 0) THROW("max_roi_height and max_roi_width cannot be negative")
        context->master_graph->to_tensor(out_ptr, static_cast<RocalTensorlayout>(tensor_format), multiplier0, multiplier1, multiplier2, offset0, offset1,
                                         offset2, reverse_channels, static_cast<RocalTensorDataType>(tensor_output_type), (unsigned)max_roi_height,
                                         (unsigned)max_roi_width);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

/* ------------------------------------------------------------------ bounding boxes */

RocalStatus rocalEnableBoundingBoxes(RocalContext p_context) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        context->master_graph->enable_meta_data();
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

RocalStatus rocalSetBoundingBoxes(RocalContext p_context, const unsigned *counts, const float *ltrb, const int *labels) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto *context = static_cast<Context *>(p_context);
    try {
        if (!context->master_graph->meta_data_enabled()) THROW("rocalEnableBoundingBoxes was not called")
        if (!counts || !ltrb || !labels) THROW("counts, box and label arrays are required")
        const size_t n = context->master_graph->batch_size();
        auto batch = std::make_shared<MetaDataBatch>(n);
        size_t k = 0;
        for (size_t i = 0; i < n; i++)
            for (unsigned j = 0; j < counts[i]; j++, k++) {
                batch->get_bb_cords_batch()[i].push_back({ltrb[4 * k], ltrb[4 * k + 1], ltrb[4 * k + 2], ltrb[4 * k + 3]});
                batch->get_labels_batch()[i].push_back(labels[k]);
            }
        context->master_graph->set_input_meta_data(batch);
    } catch (const std::exception &e) {
        report(context, e);
        return ROCAL_RUNTIME_ERROR;
    }
    return ROCAL_OK;
}

unsigned rocalGetBoundingBoxCount(RocalContext p_context, unsigned *counts) {
    if (!p_context) return 0;
    auto meta = static_cast<Context *>(p_context)->master_graph->output_meta_data();
    if (!meta) return 0;
    unsigned total = 0;
    for (size_t i = 0; i < meta->size(); i++) {
        const unsigned c = (unsigned)meta->get_bb_cords_batch()[i].size();
        if (counts) counts[i] = c;
        total += c;
    }
    return total;
}

RocalStatus rocalGetBoundingBoxCords(RocalContext p_context, float *ltrb) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto meta = static_cast<Context *>(p_context)->master_graph->output_meta_data();
    if (!meta || !ltrb) return ROCAL_RUNTIME_ERROR;
    size_t k = 0;
    for (size_t i = 0; i < meta->size(); i++)
        for (const auto &b : meta->get_bb_cords_batch()[i]) {
            ltrb[k++] = b.l;
            ltrb[k++] = b.t;
            ltrb[k++] = b.r;
            ltrb[k++] = b.b;
        }
    return ROCAL_OK;
}

// one label per box of rocalGetBoundingBoxCords (a node that pads an empty sample with a zero box adds label 0, except
// the plain resize, which adds the box only: there the label is reported as 0 too)
RocalStatus rocalGetBoundingBoxLabel(RocalContext p_context, int *labels) {
    if (!p_context) return ROCAL_CONTEXT_INVALID;
    auto meta = static_cast<Context *>(p_context)->master_graph->output_meta_data();
    if (!meta || !labels) return ROCAL_RUNTIME_ERROR;
    size_t k = 0;
    for (size_t i = 0; i < meta->size(); i++) {
        const auto &l = meta->get_labels_batch()[i];
        for (size_t j = 0; j < meta->get_bb_cords_batch()[i].size(); j++) labels[k++] = j < l.size() ? l[j] : 0;
    }
    return ROCAL_OK;
}

/* ------------------------------------------------------------------ parameters */

void rocalSetSeed(unsigned seed) { ParameterFactory::instance()->set_seed(seed); }
unsigned rocalGetSeed() { return ParameterFactory::instance()->get_seed(); }
int rocalGetIntValue(RocalIntParam p) { return I(p)->core->get(); }
float rocalGetFloatValue(RocalFloatParam p) { return F(p)->core->get(); }
RocalIntParam rocalCreateIntUniformRand(int start, int end) { return ParameterFactory::instance()->create_uniform_int_rand_param(start, end); }
RocalFloatParam rocalCreateFloatUniformRand(float start, float end) { return ParameterFactory::instance()->create_uniform_float_rand_param(start, end); }
RocalFloatParam rocalCreateFloatParameter(float val) { return ParameterFactory::instance()->create_single_value_float_param(val); }
RocalIntParam rocalCreateIntParameter(int val) { return ParameterFactory::instance()->create_single_value_int_param(val); }
RocalIntParam rocalCreateIntRand(const int *values, const double *frequencies, unsigned size) {
    return ParameterFactory::instance()->create_custom_int_rand_param(values, frequencies, size);
}
RocalFloatParam rocalCreateFloatRand(const float *values, const double *frequencies, unsigned size) {
    return ParameterFactory::instance()->create_custom_float_rand_param(values, frequencies, size);
}

namespace {
template <typename Derived, typename Wrapper, typename Fn>
RocalStatus update_param(Wrapper *w, RocalParameterType expected, Fn fn) {
    if (!w || w->type != expected) return ROCAL_INVALID_PARAMETER_TYPE;
    auto *obj = dynamic_cast<Derived *>(w->core);
    if (!obj) return ROCAL_INVALID_PARAMETER_TYPE;
    return fn(obj) == 0 ? ROCAL_OK : ROCAL_UPDATE_PARAMETER_FAILED;
}
}  // namespace

RocalStatus rocalUpdateIntUniformRand(int start, int end, RocalIntParam p) {
    return update_param<UniformRand<int>>(I(p), RocalParameterType::RANDOM_UNIFORM, [&](auto *o) { return o->update(start, end); });
}
RocalStatus rocalUpdateFloatUniformRand(float start, float end, RocalFloatParam p) {
    return update_param<UniformRand<float>>(F(p), RocalParameterType::RANDOM_UNIFORM, [&](auto *o) { return o->update(start, end); });
}
RocalStatus rocalUpdateFloatParameter(float v, RocalFloatParam p) {
    return update_param<SimpleParameter<float>>(F(p), RocalParameterType::DETERMINISTIC, [&](auto *o) { return o->update(v); });
}
RocalStatus rocalUpdateIntParameter(int v, RocalIntParam p) {
    return update_param<SimpleParameter<int>>(I(p), RocalParameterType::DETERMINISTIC, [&](auto *o) { return o->update(v); });
}
RocalStatus rocalUpdateIntRand(const int *values, const double *frequencies, unsigned size, RocalIntParam p) {
    return update_param<CustomRand<int>>(I(p), RocalParameterType::RANDOM_CUSTOM, [&](auto *o) { return o->update(values, frequencies, size); });
}
RocalStatus rocalUpdateFloatRand(const float *values, const double *frequencies, unsigned size, RocalFloatParam p) {
    return update_param<CustomRand<float>>(F(p), RocalParameterType::RANDOM_CUSTOM, [&](auto *o) { return o->update(values, frequencies, size); });
}

/* ------------------------------------------------------------------ resize family */

namespace {

// rocal_api_augmentation.cpp:449-505: which size the node is given and how large the padded output is.
constexpr float MAX_ASPECT_RATIO = 6.0f;  // rocAL/include/pipeline/commons.h:39

struct ResizePlan {
    unsigned out_w, out_h, max_w, max_h;
    RocalResizeScalingMode mode;
    std::vector<unsigned> maximum_size;
    const char *error = nullptr;
};

ResizePlan plan_resize(Tensor *input, unsigned dest_width, unsigned dest_height, RocalResizeScalingMode scaling_mode, const std::vector<unsigned> &max_size,
                       unsigned resize_shorter, unsigned resize_longer) {
    ResizePlan p{};
    if ((dest_width | dest_height | resize_longer | resize_shorter) == 0) {
        p.error = "Atleast one size 'dest_width' or 'dest_height' or 'resize_shorter' or 'resize_longer' must be specified";
        return p;
    }
    if ((dest_width | dest_height) && (resize_longer | resize_shorter)) {
        p.error = "Only one method of specifying size can be used \ndest_width and/or dest_height\nresize_shorter\nresize_longer";
        return p;
    }
    if (resize_longer && resize_shorter) {
        p.error = "'resize_longer' and 'resize_shorter' cannot be passed together. They are mutually exclusive.";
        return p;
    }
    if (resize_shorter) {
        p.mode = ROCAL_SCALING_MODE_NOT_SMALLER;
        p.out_w = p.out_h = resize_shorter;
    } else if (resize_longer) {
        p.mode = ROCAL_SCALING_MODE_NOT_LARGER;
        p.out_w = p.out_h = resize_longer;
    } else {
        p.mode = scaling_mode;
        p.out_w = dest_width;
        p.out_h = dest_height;
    }
    if (max_size.size() == 1)
        p.maximum_size = {max_size[0], max_size[0]};
    else if (max_size.size() == 2)
        p.maximum_size = {max_size[0], max_size[1]};
    else if (max_size.size() > 2) {
        p.error = "The length of max_size vector exceeds the image dimension.";
        return p;
    }
    if (p.maximum_size.size() && p.maximum_size[0] != 0 && p.maximum_size[1] != 0) {
        p.max_w = p.maximum_size[0];
        p.max_h = p.maximum_size[1];
    } else {
        if (p.mode == ROCAL_SCALING_MODE_STRETCH) {
            p.max_w = p.out_w ? p.out_w : (unsigned)input->info().max_shape()[0];
            p.max_h = p.out_h ? p.out_h : (unsigned)input->info().max_shape()[1];
        } else if (p.mode == ROCAL_SCALING_MODE_NOT_SMALLER) {
            p.max_w = (p.out_w ? p.out_w : p.out_h) * MAX_ASPECT_RATIO;
            p.max_h = (p.out_h ? p.out_h : p.out_w) * MAX_ASPECT_RATIO;
        } else {
            p.max_w = p.out_w ? p.out_w : p.out_h * MAX_ASPECT_RATIO;
            p.max_h = p.out_h ? p.out_h : p.out_w * MAX_ASPECT_RATIO;
        }
        if (p.maximum_size.size() == 2) {
            p.max_w = p.maximum_size[0] ? p.maximum_size[0] : p.max_w;
            p.max_h = p.maximum_size[1] ? p.maximum_size[1] : p.max_h;
        }
    }
    return p;
}

}  // namespace

RocalTensor rocalResize(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, RocalResizeScalingMode scaling_mode,
                        std::vector<unsigned> max_size, unsigned resize_shorter, unsigned resize_longer, RocalResizeInterpolationType interpolation_type,
                        RocalTensorLayout layout, RocalTensorOutputType dtype) {
    if (!c || !in) return add_op<ResizeNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [](ResizeNode &) {});
    ResizePlan p = plan_resize(static_cast<Tensor *>(in), dest_width, dest_height, scaling_mode, max_size, resize_shorter, resize_longer);
    return add_op<ResizeNode>(c, in, is_output, layout, dtype, Dims::SET, p.max_w, p.max_h, p.error,
                              [&](ResizeNode &n) { n.init(p.out_w, p.out_h, p.mode, p.maximum_size, interpolation_type); });
}

RocalTensor rocalResizeMirrorNormalize(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, std::vector<float> &mean,
                                       std::vector<float> &std_dev, bool is_output, RocalResizeScalingMode scaling_mode, std::vector<unsigned> max_size,
                                       unsigned resize_shorter, unsigned resize_longer, RocalResizeInterpolationType interpolation_type, RocalIntParam mirror,
                                       RocalTensorLayout layout, RocalTensorOutputType dtype) {
    if (!c || !in) return add_op<ResizeMirrorNormalizeNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [](ResizeMirrorNormalizeNode &) {});
    ResizePlan p = plan_resize(static_cast<Tensor *>(in), dest_width, dest_height, scaling_mode, max_size, resize_shorter, resize_longer);
    return add_op<ResizeMirrorNormalizeNode>(c, in, is_output, layout, dtype, Dims::SET, p.max_w, p.max_h, p.error, [&](ResizeMirrorNormalizeNode &n) {
        n.init(p.out_w, p.out_h, p.mode, p.maximum_size, interpolation_type, mean, std_dev, I(mirror));
    });
}

RocalTensor rocalCropResize(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, RocalFloatParam area,
                            RocalFloatParam aspect_ratio, RocalFloatParam x_center_drift, RocalFloatParam y_center_drift, RocalTensorLayout layout,
                            RocalTensorOutputType dtype) {
    const char *err = (dest_width == 0 || dest_height == 0) ? "CropResize node needs tp receive non-zero destination dimensions" : nullptr;
    return add_op<CropResizeNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, err,
                                  [&](CropResizeNode &n) { n.init(F(area), F(aspect_ratio), F(x_center_drift), F(y_center_drift)); });
}

RocalTensor rocalCropResizeFixed(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, float area, float aspect_ratio,
                                 float x_center_drift, float y_center_drift, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    const char *err = (dest_width == 0 || dest_height == 0) ? "CropResize node needs tp receive non-zero destination dimensions" : nullptr;
    return add_op<CropResizeNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, err,
                                  [&](CropResizeNode &n) { n.init(area, aspect_ratio, x_center_drift, y_center_drift); });
}

RocalTensor rocalROIResize(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, unsigned roi_h, unsigned roi_w,
                           float roi_pos_x, float roi_pos_y, RocalResizeInterpolationType interpolation_type, RocalTensorLayout layout,
                           RocalTensorOutputType dtype) {
    const char *err = (dest_width == 0 || dest_height == 0) ? "ROI Resize needs to receive non-zero destination dimensions" : nullptr;
    return add_op<CropResizeNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, err,
                                  [&](CropResizeNode &n) { n.init(roi_h, roi_w, roi_pos_x, roi_pos_y, interpolation_type); });
}

RocalTensor rocalResizeCropMirrorFixed(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, unsigned crop_h,
                                       unsigned crop_w, RocalIntParam mirror, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    const char *err = (dest_width == 0 || dest_height == 0) ? "Crop Mirror node needs tp receive non-zero destination dimensions" : nullptr;
    return add_op<ResizeCropMirrorNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, err,
                                        [&](ResizeCropMirrorNode &n) { n.init(crop_h, crop_w, I(mirror), ROCAL_LINEAR_INTERPOLATION); });
}

RocalTensor rocalResizeCropMirror(RocalContext c, RocalTensor in, unsigned dest_width, unsigned dest_height, bool is_output, RocalFloatParam crop_height,
                                  RocalFloatParam crop_width, RocalIntParam mirror, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    const char *err = (dest_width == 0 || dest_height == 0) ? "Crop Mirror node needs tp receive non-zero destination dimensions" : nullptr;
    return add_op<ResizeCropMirrorNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, err, [&](ResizeCropMirrorNode &n) {
        n.init(F(crop_height), F(crop_width), I(mirror), ROCAL_LINEAR_INTERPOLATION);
    });
}

/* ------------------------------------------------------------------ crop / flip / CMN */

RocalTensor rocalCropMirrorNormalize(RocalContext c, RocalTensor in, unsigned crop_height, unsigned crop_width, float start_x, float start_y,
                                     std::vector<float> &mean, std::vector<float> &std_dev, bool is_output, RocalIntParam mirror, RocalTensorLayout layout,
                                     RocalTensorOutputType dtype) {
    const char *err = (crop_width == 0 || crop_height == 0) ? "Null values passed as input" : nullptr;
    return add_op<CropMirrorNormalizeNode>(c, in, is_output, layout, dtype, Dims::SET, crop_width, crop_height, err, [&](CropMirrorNormalizeNode &n) {
        n.init(crop_height, crop_width, start_x, start_y, mean, std_dev, I(mirror));
    });
}

RocalTensor rocalCrop(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam crop_width, RocalFloatParam crop_height, RocalFloatParam,
                      RocalFloatParam crop_pos_x, RocalFloatParam crop_pos_y, RocalFloatParam, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<CropNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr,
                            [&](CropNode &n) { n.init(F(crop_height), F(crop_width), F(crop_pos_x), F(crop_pos_y)); });
}

RocalTensor rocalCropFixed(RocalContext c, RocalTensor in, unsigned crop_width, unsigned crop_height, unsigned, bool is_output, float crop_pos_x,
                           float crop_pos_y, float, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    const char *err = (crop_width == 0 || crop_height == 0) ? "Crop node needs to receive non-zero destination dimensions" : nullptr;
    return add_op<CropNode>(c, in, is_output, layout, dtype, Dims::SET, crop_width, crop_height, err,
                            [&](CropNode &n) { n.init(crop_height, crop_width, crop_pos_x, crop_pos_y); });
}

RocalTensor rocalCropCenterFixed(RocalContext c, RocalTensor in, unsigned crop_width, unsigned crop_height, unsigned, bool is_output,
                                 RocalTensorLayout layout, RocalTensorOutputType dtype) {
    const char *err = (crop_width == 0 || crop_height == 0) ? "Crop node needs to receive non-zero destination dimensions" : nullptr;
    return add_op<CropNode>(c, in, is_output, layout, dtype, Dims::SET, crop_width, crop_height, err, [&](CropNode &n) { n.init(crop_height, crop_width); });
}

RocalTensor rocalRandomCrop(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam crop_area_factor, RocalFloatParam crop_aspect_ratio,
                            RocalFloatParam crop_pos_x, RocalFloatParam crop_pos_y, int num_of_attempts, RocalTensorLayout layout,
                            RocalTensorOutputType dtype) {
    return add_op<RandomCropNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](RandomCropNode &n) {
        n.init(F(crop_area_factor), F(crop_aspect_ratio), F(crop_pos_x), F(crop_pos_y), num_of_attempts);
    });
}

RocalTensor rocalFlip(RocalContext c, RocalTensor in, bool is_output, RocalIntParam h, RocalIntParam v, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<FlipNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](FlipNode &n) { n.init(I(h), I(v)); });
}

RocalTensor rocalFlipFixed(RocalContext c, RocalTensor in, int h, int v, bool is_output, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<FlipNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](FlipNode &n) { n.init(h, v); });
}

/* ------------------------------------------------------------------ colour family */

RocalTensor rocalBrightness(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam alpha, RocalFloatParam beta, RocalTensorLayout layout,
                            RocalTensorOutputType dtype) {
    return add_op<BrightnessNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](BrightnessNode &n) { n.init(F(alpha), F(beta)); });
}
RocalTensor rocalBrightnessFixed(RocalContext c, RocalTensor in, float alpha, float beta, bool is_output, RocalTensorLayout layout,
                                 RocalTensorOutputType dtype) {
    return add_op<BrightnessNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](BrightnessNode &n) { n.init(alpha, beta); });
}
RocalTensor rocalContrast(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam factor, RocalFloatParam center, RocalTensorLayout layout,
                          RocalTensorOutputType dtype) {
    return add_op<ContrastNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](ContrastNode &n) { n.init(F(factor), F(center)); });
}
RocalTensor rocalContrastFixed(RocalContext c, RocalTensor in, float factor, float center, bool is_output, RocalTensorLayout layout,
                               RocalTensorOutputType dtype) {
    return add_op<ContrastNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](ContrastNode &n) { n.init(factor, center); });
}
RocalTensor rocalHue(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam hue, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<HueNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](HueNode &n) { n.init(F(hue)); });
}
RocalTensor rocalHueFixed(RocalContext c, RocalTensor in, float hue, bool is_output, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<HueNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](HueNode &n) { n.init(hue); });
}
RocalTensor rocalSaturation(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam sat, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<SaturationNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](SaturationNode &n) { n.init(F(sat)); });
}
RocalTensor rocalSaturationFixed(RocalContext c, RocalTensor in, float sat, bool is_output, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<SaturationNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](SaturationNode &n) { n.init(sat); });
}
RocalTensor rocalGamma(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam gamma, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<GammaNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](GammaNode &n) { n.init(F(gamma)); });
}
RocalTensor rocalGammaFixed(RocalContext c, RocalTensor in, float gamma, bool is_output, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<GammaNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](GammaNode &n) { n.init(gamma); });
}
// rocal_api_augmentation.cpp:2288-2308: same shape and layout as the input, the requested type
RocalTensor rocalNormalize(RocalContext c, RocalTensor in, std::vector<unsigned> &axes, std::vector<float> &mean, std::vector<float> &std_dev, bool is_output,
                           float scale, float shift, RocalTensorOutputType dtype) {
    const auto layout = in ? (RocalTensorLayout) static_cast<Tensor *>(in)->info().layout() : ROCAL_NHWC;
    return add_op<NormalizeNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](NormalizeNode &n) { n.init(axes, mean, std_dev, scale, shift); });
}

// rocal_api_augmentation.cpp:2349-2378: the dims follow the permutation, the layout is the one asked for
RocalTensor rocalTranspose(RocalContext c, RocalTensor in, std::vector<unsigned> perm, bool is_output, RocalTensorLayout output_layout) {
    const char *err = nullptr;
    unsigned w = 0, h = 0;
    if (c && in) {
        const TensorInfo &info = static_cast<Tensor *>(in)->info();
        if (perm.size() != 3) {
            err = "Transpose permutation must match with the input dims";
        } else {
            const bool swap = (perm == std::vector<unsigned>{2, 1, 0}) || (perm == std::vector<unsigned>{1, 0, 2});
            w = (unsigned)(swap ? info.max_shape()[1] : info.max_shape()[0]);
            h = (unsigned)(swap ? info.max_shape()[0] : info.max_shape()[1]);
        }
    }
    const auto dtype = in ? (RocalTensorOutputType) static_cast<Tensor *>(in)->info().data_type() : ROCAL_UINT8;
    return add_op<TransposeNode>(c, in, is_output, output_layout, dtype, Dims::SET, w, h, err, [&](TransposeNode &n) { n.init(perm); });
}

RocalTensor rocalExposure(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam exposure_factor, RocalTensorLayout layout,
                          RocalTensorOutputType dtype) {
    return add_op<ExposureNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](ExposureNode &n) { n.init(F(exposure_factor)); });
}
RocalTensor rocalExposureFixed(RocalContext c, RocalTensor in, float exposure_factor, bool is_output, RocalTensorLayout layout,
                               RocalTensorOutputType dtype) {
    return add_op<ExposureNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](ExposureNode &n) { n.init(exposure_factor); });
}
RocalTensor rocalColorTemp(RocalContext c, RocalTensor in, bool is_output, RocalIntParam adjustment, RocalTensorLayout layout,
                           RocalTensorOutputType dtype) {
    return add_op<ColorTemperatureNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr,
                                        [&](ColorTemperatureNode &n) { n.init(I(adjustment)); });
}
RocalTensor rocalColorTempFixed(RocalContext c, RocalTensor in, int adjustment, bool is_output, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<ColorTemperatureNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr,
                                        [&](ColorTemperatureNode &n) { n.init(adjustment); });
}
RocalTensor rocalBlend(RocalContext c, RocalTensor in1, RocalTensor in2, bool is_output, RocalFloatParam ratio, RocalTensorLayout layout,
                       RocalTensorOutputType dtype) {
    return add_op<BlendNode>(c, in1, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](BlendNode &n) { n.init(F(ratio)); }, in2, true);
}
RocalTensor rocalBlendFixed(RocalContext c, RocalTensor in1, RocalTensor in2, float ratio, bool is_output, RocalTensorLayout layout,
                            RocalTensorOutputType dtype) {
    return add_op<BlendNode>(c, in1, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](BlendNode &n) { n.init(ratio); }, in2, true);
}
RocalTensor rocalColorTwist(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam alpha, RocalFloatParam beta, RocalFloatParam hue,
                            RocalFloatParam sat, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    return add_op<ColorTwistNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr,
                                  [&](ColorTwistNode &n) { n.init(F(alpha), F(beta), F(hue), F(sat)); });
}
RocalTensor rocalColorTwistFixed(RocalContext c, RocalTensor in, float alpha, float beta, float hue, float sat, bool is_output, RocalTensorLayout layout,
                                 RocalTensorOutputType dtype) {
    return add_op<ColorTwistNode>(c, in, is_output, layout, dtype, Dims::KEEP, 0, 0, nullptr, [&](ColorTwistNode &n) { n.init(alpha, beta, hue, sat); });
}

/* ------------------------------------------------------------------ warp affine / rotate */

namespace {
void default_dims(RocalTensor in, unsigned &w, unsigned &h) {
    if (in && (w == 0 || h == 0)) {
        w = (unsigned)static_cast<Tensor *>(in)->info().max_shape()[0];
        h = (unsigned)static_cast<Tensor *>(in)->info().max_shape()[1];
    }
}
}  // namespace

RocalTensor rocalRotate(RocalContext c, RocalTensor in, bool is_output, RocalFloatParam angle, unsigned dest_width, unsigned dest_height,
                        RocalResizeInterpolationType interpolation_type, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    default_dims(in, dest_width, dest_height);
    return add_op<RotateNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, nullptr,
                              [&](RotateNode &n) { n.init(F(angle), interpolation_type); });
}
RocalTensor rocalRotateFixed(RocalContext c, RocalTensor in, float angle, bool is_output, unsigned dest_width, unsigned dest_height,
                             RocalResizeInterpolationType interpolation_type, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    default_dims(in, dest_width, dest_height);
    return add_op<RotateNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, nullptr,
                              [&](RotateNode &n) { n.init(angle, interpolation_type); });
}
RocalTensor rocalWarpAffine(RocalContext c, RocalTensor in, bool is_output, unsigned dest_height, unsigned dest_width, RocalFloatParam x0,
                            RocalFloatParam x1, RocalFloatParam y0, RocalFloatParam y1, RocalFloatParam o0, RocalFloatParam o1,
                            RocalResizeInterpolationType interpolation_type, RocalTensorLayout layout, RocalTensorOutputType dtype) {
    default_dims(in, dest_width, dest_height);
    return add_op<WarpAffineNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, nullptr, [&](WarpAffineNode &n) {
        n.init(F(x0), F(x1), F(y0), F(y1), F(o0), F(o1), interpolation_type);
    });
}
RocalTensor rocalWarpAffineFixed(RocalContext c, RocalTensor in, float x0, float x1, float y0, float y1, float o0, float o1, bool is_output,
                                 unsigned dest_height, unsigned dest_width, RocalResizeInterpolationType interpolation_type, RocalTensorLayout layout,
                                 RocalTensorOutputType dtype) {
    default_dims(in, dest_width, dest_height);
    return add_op<WarpAffineNode>(c, in, is_output, layout, dtype, Dims::SET, dest_width, dest_height, nullptr,
                                  [&](WarpAffineNode &n) { n.init(x0, x1, y0, y1, o0, o1, interpolation_type); });
}
