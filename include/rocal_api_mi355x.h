// rocal_api_mi355x.h - public host API of the MI355X augmentation hot path: the rocAL C API entry points of the hot-path
// operators with the reference's names, argument order, defaults and error behaviour (rocAL/include/api/rocal_api.h:83-110,
// rocal_api_parameters.h:39-161, rocal_api_augmentation.h, rocal_api_info.h:106, rocal_api_data_transfer.h:45-66), so that a
// program written against rocAL's headers for these operators compiles against this one and links with
// librocal_mi355x_host.so. Like the reference's, these are extern "C" names with C++ types (std::vector, default arguments).
// This header is self-contained: it includes nothing of the library's internals.
//
// Loaders, decoders and the output ring buffer are not part of the hot path. Where the reference would create a source
// with a reader + decoder, this API takes decoded batches that already sit in device memory:
//   rocalDeviceSource()      declares the input tensor (u8 RGB, NHWC, padded to max_height x max_width)
//   rocalDeviceSourceFeed()  hands the next batch: device pointer + per-sample width/height
// and an output is read as in the reference, through rocalGetOutputTensors(ctx)->at(i)->copy_data(...) / ->buffer() /
// ->copy_roi(...) (rocal_api_tensor.h:38-93, rocal_api_data_transfer.h:43,83), or written straight into memory the caller owns
// (rocalTensor::set_mem_handle / rocalTensorSetBuffer, e.g. the data pointer of a torch tensor).
//
// rocalRun() enqueues the batch on the context's stream and returns; the wait for it is where the consumer takes the
// result: rocalGetOutputTensors, rocalTensor::copy_data / buffer, rocalCopyToOutput, rocalToTensor and rocalTensorBuffer
// return only when the batch is complete (the reference separates producer and consumer the same way, through its output
// ring buffer: ring_buffer.cpp:118-119, master_graph.cpp:1019-1043). A consumer that works on a HIP stream of its own
// can make that stream wait instead of the host: rocalOutputsWaitOnStream.
#ifndef ROCAL_API_MI355X_H
#define ROCAL_API_MI355X_H
#include <cstddef>
#include <cstdint>
#include <vector>

// rocAL/include/api/rocal_api_types.h:326-366
enum RocalResizeScalingMode {
    ROCAL_SCALING_MODE_DEFAULT = 0,
    ROCAL_SCALING_MODE_STRETCH = 1,
    ROCAL_SCALING_MODE_NOT_SMALLER = 2,
    ROCAL_SCALING_MODE_NOT_LARGER = 3,
    ROCAL_SCALING_MODE_MIN_MAX = 4
};
enum RocalResizeInterpolationType {
    ROCAL_NEAREST_NEIGHBOR_INTERPOLATION = 0,
    ROCAL_LINEAR_INTERPOLATION = 1,
    ROCAL_CUBIC_INTERPOLATION = 2,
    ROCAL_LANCZOS_INTERPOLATION = 3,
    ROCAL_GAUSSIAN_INTERPOLATION = 4,
    ROCAL_TRIANGULAR_INTERPOLATION = 5
};

#define ROCAL_API_CALL __attribute__((visibility("default")))

typedef void *RocalContext;
typedef void *RocalFloatParam;
typedef void *RocalIntParam;

// rocAL/include/api/rocal_api_types.h:112-128,151-158,208-268,372-391
enum RocalStatus { ROCAL_OK = 0, ROCAL_CONTEXT_INVALID, ROCAL_RUNTIME_ERROR, ROCAL_UPDATE_PARAMETER_FAILED, ROCAL_INVALID_PARAMETER_TYPE };
enum RocalProcessMode { ROCAL_PROCESS_GPU = 0, ROCAL_PROCESS_CPU = 1 };
enum RocalTensorLayout { ROCAL_NHWC = 0, ROCAL_NCHW = 1, ROCAL_NONE = 9 };
enum RocalTensorOutputType { ROCAL_FP32 = 0, ROCAL_FP16 = 1, ROCAL_UINT8 = 2 };
enum RocalOutputMemType { ROCAL_MEMCPY_HOST = 0, ROCAL_MEMCPY_GPU = 1, ROCAL_MEMCPY_PINNED = 2 };
enum RocalTensorBackend { ROCAL_CPU = 0, ROCAL_GPU = 1 };
enum class RocalROICordsType { ROCAL_LTRB = 0, ROCAL_XYWH = 1 };

/* ---- tensors (rocAL/include/api/rocal_api_tensor.h:38-93): the reference's abstract classes, member for member. Every
   augmentation entry point takes and returns a RocalTensor; the tensors of a context live until rocalRelease.
     buffer()         device address of the tensor's batch (waits for the batch that is being computed);
     copy_data(p, t)  copies data_size() bytes to p: device memory for ROCAL_MEMCPY_GPU, host (pageable or pinned) memory for
                      ROCAL_MEMCPY_HOST / ROCAL_MEMCPY_PINNED; returns 0 (tensor.cpp:419-454);
     copy_data(p, x, y, cols, rows)  the window at (x, y) of every sample's first plane, densely packed, to host memory
                      (tensor.cpp:456-476 reads host memory there; this build copies from the device);
     dims()/strides() in the order of the layout ({N,H,W,C} or {N,C,H,W}), strides in bytes (tensor.h:250-255);
     shape()          {max_width, max_height};  copy_roi(p): 4 unsigned per sample, x y w h (get_roi_dims_size() == 2);
     set_mem_handle(p) the node that produces the tensor writes to p from the next run on (16-byte aligned device memory). ---- */
class rocalTensor {
   public:
    virtual ~rocalTensor() = default;
    virtual void *buffer() = 0;
    virtual unsigned copy_data(void *user_buffer, RocalOutputMemType external_mem_type = ROCAL_MEMCPY_HOST) = 0;
    virtual unsigned copy_data(void *user_buffer, unsigned int x_offset, unsigned int y_offset, unsigned int max_cols, unsigned int max_rows) = 0;
    virtual unsigned num_of_dims() = 0;
    virtual unsigned batch_size() = 0;
    virtual std::vector<size_t> dims() = 0;
    virtual std::vector<size_t> strides() = 0;
    virtual RocalTensorLayout layout() = 0;
    virtual RocalTensorBackend backend() = 0;
    virtual RocalTensorOutputType data_type() = 0;
    virtual RocalOutputMemType mem_type() = 0;
    virtual size_t data_size() = 0;
    virtual RocalROICordsType roi_type() = 0;
    virtual size_t get_roi_dims_size() = 0;
    virtual void copy_roi(void *roi_buffer) = 0;
    virtual std::vector<size_t> shape() = 0;
    virtual void set_dims(std::vector<size_t> dims) = 0;
    virtual void set_mem_handle(void *buffer) = 0;
    virtual void set_tensor_layout(RocalTensorLayout layout) = 0;
    virtual uint64_t data_type_size() = 0;
};
class rocalTensorList {
   public:
    virtual ~rocalTensorList() = default;
    virtual uint64_t size() = 0;
    virtual rocalTensor *at(size_t index) = 0;
};
typedef rocalTensor *RocalTensor;
typedef rocalTensorList *RocalTensorList;

/* ---- context (rocal_api.h:83-110). Only ROCAL_PROCESS_GPU exists: there is no CPU path. ---- */
extern "C" RocalContext ROCAL_API_CALL rocalCreate(size_t batch_size, RocalProcessMode affinity, int gpu_id = 0, size_t cpu_thread_count = 1,
                                                   size_t prefetch_queue_depth = 3, RocalTensorOutputType output_tensor_data_type = ROCAL_FP32);
extern "C" RocalStatus ROCAL_API_CALL rocalVerify(RocalContext context);
extern "C" RocalStatus ROCAL_API_CALL rocalRun(RocalContext context);
extern "C" RocalStatus ROCAL_API_CALL rocalRelease(RocalContext context);
extern "C" const char *ROCAL_API_CALL rocalGetErrorMessage(RocalContext context);
// Which neighbour the bilinear kernels take at the right / lower edge of a source window (no counterpart in the reference's
// API; call it before the first resize node is added). 0, the default: the last pixel of the window (the textbook rule).
// 1: the last-but-one, as the reference's own device kernel clamps (rocAL/rocAL_hip/rocal_hip_kernels.cpp:339-345,356-362).
// The environment variable ROCAL_BILINEAR_EDGE (0 / 1, or "device") sets the default that rocalCreate starts from.
extern "C" RocalStatus ROCAL_API_CALL rocalSetBilinearEdgeRule(RocalContext context, int device_rule);

/* ---- timing (rocal_api_info.h:106, rocal_api_types.h:79-84): microseconds accumulated since the last call, which resets them.
   process_time brackets Graph::process() as the reference's does (master_graph.cpp:1015-1017): the launches of a batch and the
   wait for them; transfer_time is the time spent in rocalToTensor; load and decode time belong to the loaders and stay 0.
   rocalGetParameterUpdateTime (no counterpart in the reference) gives the time of the per-batch parameter renewal and node updates
   that run before process() on the same thread (master_graph.cpp:408,1010-1013). ---- */
struct TimingInfo {
    long long unsigned load_time;
    long long unsigned decode_time;
    long long unsigned process_time;
    long long unsigned transfer_time;
};
extern "C" TimingInfo ROCAL_API_CALL rocalGetTimingInfo(RocalContext rocal_context);
extern "C" long long unsigned ROCAL_API_CALL rocalGetParameterUpdateTime(RocalContext rocal_context);

/* ---- decoded batches in device memory (stands where the reference's loader modules stand) ---- */
extern "C" RocalTensor ROCAL_API_CALL rocalDeviceSource(RocalContext context, unsigned max_width, unsigned max_height, bool is_output);
extern "C" RocalStatus ROCAL_API_CALL rocalDeviceSourceFeed(RocalContext context, RocalTensor source, const void *device_ptr, const unsigned *roi_width,
                                                            const unsigned *roi_height);
// A source fed by a loader through a ring of PACKED batches (stands where the loader's CircularBuffer and its padded
// [N, Hmax, Wmax, 3] staging stand: rocAL/source/loaders/circular_buffer.cpp:88-160, image_read_and_decode.cpp:165-390).
// The loader places every decoded image of a batch into pinned host memory (rocalPackedSourcePlaceImage returns where the
// image's first row goes and the row stride to use: width*3 rounded up to a multiple of 4) and pushes the batch, which starts
// ONE asynchronous copy of the bytes written; rocalRun() consumes the oldest pushed batch of every packed source.
// queue_depth slots (>= 2) of slot_bytes each (0: every image at max size). Place and push may run on a loader thread while
// another thread calls rocalRun: place blocks while the ring is full.
extern "C" RocalTensor ROCAL_API_CALL rocalPackedSource(RocalContext context, unsigned max_width, unsigned max_height, bool is_output,
                                                        unsigned queue_depth, size_t slot_bytes);
extern "C" unsigned char *ROCAL_API_CALL rocalPackedSourcePlaceImage(RocalContext context, RocalTensor source, unsigned index, unsigned width,
                                                                     unsigned height, unsigned *row_stride);
extern "C" RocalStatus ROCAL_API_CALL rocalPackedSourcePush(RocalContext context, RocalTensor source);
// Blocks the caller until a pushed batch is waiting (the consumer side of a loader thread); rocalRun() on an empty ring
// returns an error instead of blocking.
extern "C" RocalStatus ROCAL_API_CALL rocalPackedSourceWait(RocalContext context, RocalTensor source);
extern "C" size_t ROCAL_API_CALL rocalPackedSourceLevel(RocalContext context, RocalTensor source);
// Shut-down of the ring, as the reference's loaders do it (image_loader.cpp:84,126-127: unblock_writer / unblock_reader):
// wakes a loader thread blocked in rocalPackedSourcePlaceImage and a consumer blocked in rocalPackedSourceWait; they and
// every later caller get an error ("released") instead of a slot. rocalRelease does this for every packed source and frees
// the slots only when no thread is inside one of these calls any more.
extern "C" RocalStatus ROCAL_API_CALL rocalPackedSourceStop(RocalContext context, RocalTensor source);
/* ---- flat getters over the same tensors for callers without C++ (ctypes): extras, not in the reference ---- */
extern "C" void *ROCAL_API_CALL rocalTensorBuffer(RocalTensor tensor);
// Binds an output tensor to device memory the caller owns (at least rocalTensorDataSize bytes, 16-byte aligned), before or
// after rocalVerify and as often as wanted between runs: the node that produces the tensor writes there directly. Stands where
// the reference copies a finished output into the framework's tensor (rocalTensor::copy_data, rocAL/source/pipeline/tensor.cpp:419-454,
// called from rocAL_pybind/amd/rocal/plugin/pytorch.py:118-135).
extern "C" RocalStatus ROCAL_API_CALL rocalTensorSetBuffer(RocalContext context, RocalTensor tensor, void *device_ptr);
// x,y,w,h per sample
extern "C" const unsigned *ROCAL_API_CALL rocalTensorRoi(RocalTensor tensor);
extern "C" size_t ROCAL_API_CALL rocalTensorDataSize(RocalTensor tensor);
// Padded dimensions in the order of the layout ({N,H,W,C} or {N,C,H,W}), layout and data type of a tensor
// (rocalTensor::dims / layout / data_type, rocAL/include/api/rocal_api_tensor.h:60-90).
extern "C" RocalStatus ROCAL_API_CALL rocalTensorInfo(RocalTensor tensor, size_t dims[4], int *layout, int *data_type);

/* ---- tensors the caller wants to read after a run (rocal_api_data_transfer.h:75): called before rocalVerify, as the Python
   pipeline does for what define_graph returns; a tensor created with is_output = true is an output already. ---- */
extern "C" void ROCAL_API_CALL rocalSetOutputs(RocalContext p_context, unsigned int num_of_outputs, std::vector<RocalTensor> &output_images);

/* ---- results of the last rocalRun (rocal_api_data_transfer.h:43,83). Both wait until the batch is complete.
   rocalGetOutputTensors: the list of output tensors, owned by the context. rocalCopyToOutput: the single output tensor to
   host memory, out_size = its data_size() (master_graph.cpp:859-927). ---- */
extern "C" RocalTensorList ROCAL_API_CALL rocalGetOutputTensors(RocalContext context);
extern "C" RocalStatus ROCAL_API_CALL rocalCopyToOutput(RocalContext context, unsigned char *out_ptr, size_t out_size);
// Makes a HIP stream of the caller (hipStream_t as void *, null = the default stream) wait for the batch of the last rocalRun
// instead of the host: what a framework that consumes the output on its own stream calls (no counterpart in the reference,
// whose consumer is the host thread).
extern "C" RocalStatus ROCAL_API_CALL rocalOutputsWaitOnStream(RocalContext context, void *stream);

/* ---- u8 output -> float tensor (rocal_api_data_transfer.h:45-66). out_ptr is device memory: only ROCAL_MEMCPY_GPU exists. ---- */
extern "C" RocalStatus ROCAL_API_CALL rocalToTensor(RocalContext rocal_context, void *out_ptr, RocalTensorLayout tensor_format,
                                                    RocalTensorOutputType tensor_output_type, float multiplier0, float multiplier1, float multiplier2,
                                                    float offset0, float offset1, float offset2, bool reverse_channels,
                                                    RocalOutputMemType output_mem_type, int max_roi_height = 0, int max_roi_width = 0);

/* ---- bounding boxes (rocal_api_meta_data.h). Metadata readers are outside the hot path: rocalEnableBoundingBoxes() stands
   where rocalCreateCOCOReader() & co. stand (before the augmentations are added); the boxes of a batch (l,t,r,b in pixels
   of the decoded image, `counts[i]` per sample, all samples back to back) are handed in before rocalRun() and the
   transformed ones are read back after it, in the same layout. ---- */
extern "C" RocalStatus ROCAL_API_CALL rocalEnableBoundingBoxes(RocalContext context);
extern "C" RocalStatus ROCAL_API_CALL rocalSetBoundingBoxes(RocalContext context, const unsigned *counts, const float *ltrb, const int *labels);
extern "C" unsigned ROCAL_API_CALL rocalGetBoundingBoxCount(RocalContext context, unsigned *counts);  // returns the total
extern "C" RocalStatus ROCAL_API_CALL rocalGetBoundingBoxCords(RocalContext context, float *ltrb);
extern "C" RocalStatus ROCAL_API_CALL rocalGetBoundingBoxLabel(RocalContext context, int *labels);

/* ---- parameters (rocal_api_parameters.h:39-161) ---- */
extern "C" void ROCAL_API_CALL rocalSetSeed(unsigned seed);
extern "C" unsigned ROCAL_API_CALL rocalGetSeed();
extern "C" RocalIntParam ROCAL_API_CALL rocalCreateIntUniformRand(int start, int end);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateIntUniformRand(int start, int end, RocalIntParam updating_obj);
extern "C" int ROCAL_API_CALL rocalGetIntValue(RocalIntParam obj);
extern "C" float ROCAL_API_CALL rocalGetFloatValue(RocalFloatParam obj);
extern "C" RocalFloatParam ROCAL_API_CALL rocalCreateFloatUniformRand(float start, float end);
extern "C" RocalFloatParam ROCAL_API_CALL rocalCreateFloatParameter(float val);
extern "C" RocalIntParam ROCAL_API_CALL rocalCreateIntParameter(int val);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateFloatParameter(float new_val, RocalFloatParam input_obj);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateIntParameter(int new_val, RocalIntParam input_obj);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateFloatUniformRand(float start, float end, RocalFloatParam updating_obj);
extern "C" RocalIntParam ROCAL_API_CALL rocalCreateIntRand(const int *values, const double *frequencies, unsigned size);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateIntRand(const int *values, const double *frequencies, unsigned size, RocalIntParam updating_obj);
extern "C" RocalFloatParam ROCAL_API_CALL rocalCreateFloatRand(const float *values, const double *frequencies, unsigned size);
extern "C" RocalStatus ROCAL_API_CALL rocalUpdateFloatRand(const float *values, const double *frequencies, unsigned size, RocalFloatParam updating_obj);

/* ---- augmentations (rocal_api_augmentation.h; line of each declaration given) ---- */
extern "C" RocalTensor ROCAL_API_CALL rocalResize(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height, bool is_output,
                                                  RocalResizeScalingMode scaling_mode = ROCAL_SCALING_MODE_STRETCH, std::vector<unsigned> max_size = {},
                                                  unsigned resize_shorter = 0, unsigned resize_longer = 0,
                                                  RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                  RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :67
extern "C" RocalTensor ROCAL_API_CALL rocalResizeMirrorNormalize(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height,
                                                                 std::vector<float> &mean, std::vector<float> &std_dev, bool is_output,
                                                                 RocalResizeScalingMode scaling_mode = ROCAL_SCALING_MODE_STRETCH,
                                                                 std::vector<unsigned> max_size = {}, unsigned resize_shorter = 0, unsigned resize_longer = 0,
                                                                 RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                                 RocalIntParam mirror = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                                 RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :98
extern "C" RocalTensor ROCAL_API_CALL rocalCropResize(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height, bool is_output,
                                                      RocalFloatParam area = NULL, RocalFloatParam aspect_ratio = NULL, RocalFloatParam x_center_drift = NULL,
                                                      RocalFloatParam y_center_drift = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :125
extern "C" RocalTensor ROCAL_API_CALL rocalCropResizeFixed(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height,
                                                           bool is_output, float area, float aspect_ratio, float x_center_drift, float y_center_drift,
                                                           RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :151
extern "C" RocalTensor ROCAL_API_CALL rocalROIResize(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height, bool is_output,
                                                     unsigned roi_h, unsigned roi_w, float roi_pos_x = 0.0f, float roi_pos_y = 0.0f,
                                                     RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                     RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :175
extern "C" RocalTensor ROCAL_API_CALL rocalRotate(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam angle = NULL,
                                                  unsigned dest_width = 0, unsigned dest_height = 0,
                                                  RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                  RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :200
extern "C" RocalTensor ROCAL_API_CALL rocalRotateFixed(RocalContext context, RocalTensor input, float angle, bool is_output, unsigned dest_width = 0,
                                                       unsigned dest_height = 0, RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                       RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :220
extern "C" RocalTensor ROCAL_API_CALL rocalBrightness(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam alpha = NULL,
                                                      RocalFloatParam beta = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :237
extern "C" RocalTensor ROCAL_API_CALL rocalBrightnessFixed(RocalContext context, RocalTensor input, float alpha, float beta, bool is_output,
                                                           RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :253
extern "C" RocalTensor ROCAL_API_CALL rocalContrast(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam contrast_factor = NULL,
                                                    RocalFloatParam contrast_center = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                    RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :302
extern "C" RocalTensor ROCAL_API_CALL rocalContrastFixed(RocalContext context, RocalTensor input, float contrast_factor, float contrast_center,
                                                         bool is_output, RocalTensorLayout output_layout = ROCAL_NONE,
                                                         RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :319
extern "C" RocalTensor ROCAL_API_CALL rocalFlip(RocalContext context, RocalTensor input, bool is_output, RocalIntParam horizonal_flag = NULL,
                                                RocalIntParam vertical_flag = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :336
extern "C" RocalTensor ROCAL_API_CALL rocalFlipFixed(RocalContext context, RocalTensor input, int horizonal_flag, int vertical_flag, bool is_output,
                                                     RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :352
extern "C" RocalTensor ROCAL_API_CALL rocalWarpAffine(RocalContext context, RocalTensor input, bool is_output, unsigned dest_height = 0,
                                                      unsigned dest_width = 0, RocalFloatParam x0 = NULL, RocalFloatParam x1 = NULL,
                                                      RocalFloatParam y0 = NULL, RocalFloatParam y1 = NULL, RocalFloatParam o0 = NULL,
                                                      RocalFloatParam o1 = NULL, RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                      RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :422
extern "C" RocalTensor ROCAL_API_CALL rocalWarpAffineFixed(RocalContext context, RocalTensor input, float x0, float x1, float y0, float y1, float o0,
                                                           float o1, bool is_output, unsigned int dest_height = 0, unsigned int dest_width = 0,
                                                           RocalResizeInterpolationType interpolation_type = ROCAL_LINEAR_INTERPOLATION,
                                                           RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :449
extern "C" RocalTensor ROCAL_API_CALL rocalHue(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam hue = NULL,
                                               RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :794
extern "C" RocalTensor ROCAL_API_CALL rocalHueFixed(RocalContext context, RocalTensor input, float hue, bool is_output,
                                                    RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :810
extern "C" RocalTensor ROCAL_API_CALL rocalSaturation(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam saturation = NULL,
                                                      RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :826
extern "C" RocalTensor ROCAL_API_CALL rocalSaturationFixed(RocalContext context, RocalTensor input, float saturation, bool is_output,
                                                           RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :842
extern "C" RocalTensor ROCAL_API_CALL rocalColorTwist(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam alpha = NULL,
                                                      RocalFloatParam beta = NULL, RocalFloatParam hue = NULL, RocalFloatParam sat = NULL,
                                                      RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :878
extern "C" RocalTensor ROCAL_API_CALL rocalColorTwistFixed(RocalContext context, RocalTensor input, float alpha, float beta, float hue, float sat,
                                                           bool is_output, RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :900
extern "C" RocalTensor ROCAL_API_CALL rocalGamma(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam gamma = NULL,
                                                 RocalTensorLayout output_layout = ROCAL_NONE,
                                                 RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :269
extern "C" RocalTensor ROCAL_API_CALL rocalGammaFixed(RocalContext context, RocalTensor input, float gamma, bool is_output,
                                                      RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :285
extern "C" RocalTensor ROCAL_API_CALL rocalBlend(RocalContext context, RocalTensor input1, RocalTensor input2, bool is_output,
                                                 RocalFloatParam ratio = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                 RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :382
extern "C" RocalTensor ROCAL_API_CALL rocalBlendFixed(RocalContext context, RocalTensor input1, RocalTensor input2, float ratio, bool is_output,
                                                      RocalTensorLayout output_layout = ROCAL_NONE,
                                                      RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :399
extern "C" RocalTensor ROCAL_API_CALL rocalColorTemp(RocalContext context, RocalTensor input, bool is_output, RocalIntParam adjustment = NULL,
                                                     RocalTensorLayout output_layout = ROCAL_NONE,
                                                     RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :667
extern "C" RocalTensor ROCAL_API_CALL rocalColorTempFixed(RocalContext context, RocalTensor input, int adjustment, bool is_output,
                                                          RocalTensorLayout output_layout = ROCAL_NONE,
                                                          RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :683
extern "C" RocalTensor ROCAL_API_CALL rocalExposure(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam exposure_factor = NULL,
                                                    RocalTensorLayout output_layout = ROCAL_NONE,
                                                    RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :763
extern "C" RocalTensor ROCAL_API_CALL rocalExposureFixed(RocalContext context, RocalTensor input, float exposure_factor, bool is_output,
                                                         RocalTensorLayout output_layout = ROCAL_NONE,
                                                         RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :779
// Normalize and Transpose on image tensors (rocal_api_augmentation.h: rocalNormalize, rocalTranspose). axes / perm name the axes of
// the tensor without its batch axis: 0 height, 1 width, 2 channels. Normalize: axes {0,1} or {0,1,2}; an empty mean / std_dev is
// computed per sample. Transpose: {0,1,2}, {2,0,1}, {1,0,2}, {2,1,0} with the output layout the permutation produces.
extern "C" RocalTensor ROCAL_API_CALL rocalNormalize(RocalContext context, RocalTensor input, std::vector<unsigned> &axes, std::vector<float> &mean,
                                                     std::vector<float> &std_dev, bool is_output, float scale = 1.0, float shift = 0.0,
                                                     RocalTensorOutputType output_datatype = ROCAL_FP32);
extern "C" RocalTensor ROCAL_API_CALL rocalTranspose(RocalContext context, RocalTensor input, std::vector<unsigned> perm, bool is_output,
                                                     RocalTensorLayout output_layout = ROCAL_NONE);
extern "C" RocalTensor ROCAL_API_CALL rocalCropMirrorNormalize(RocalContext context, RocalTensor input, unsigned crop_height, unsigned crop_width,
                                                               float start_x, float start_y, std::vector<float> &mean, std::vector<float> &std_dev,
                                                               bool is_output, RocalIntParam mirror = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                               RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :925
extern "C" RocalTensor ROCAL_API_CALL rocalCrop(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam crop_width = NULL,
                                                RocalFloatParam crop_height = NULL, RocalFloatParam crop_depth = NULL, RocalFloatParam crop_pox_x = NULL,
                                                RocalFloatParam crop_pos_y = NULL, RocalFloatParam crop_pos_z = NULL,
                                                RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :952
extern "C" RocalTensor ROCAL_API_CALL rocalCropFixed(RocalContext context, RocalTensor input, unsigned crop_width, unsigned crop_height,
                                                     unsigned crop_depth, bool is_output, float crop_pox_x, float crop_pos_y, float crop_pos_z,
                                                     RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :977
extern "C" RocalTensor ROCAL_API_CALL rocalCropCenterFixed(RocalContext context, RocalTensor input, unsigned crop_width, unsigned crop_height,
                                                           unsigned crop_depth, bool is_output, RocalTensorLayout output_layout = ROCAL_NONE,
                                                           RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :1000
extern "C" RocalTensor ROCAL_API_CALL rocalResizeCropMirrorFixed(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height,
                                                                 bool is_output, unsigned crop_h, unsigned crop_w, RocalIntParam mirror,
                                                                 RocalTensorLayout output_layout = ROCAL_NONE,
                                                                 RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :1022
extern "C" RocalTensor ROCAL_API_CALL rocalResizeCropMirror(RocalContext context, RocalTensor input, unsigned dest_width, unsigned dest_height,
                                                            bool is_output, RocalFloatParam crop_height = NULL, RocalFloatParam crop_width = NULL,
                                                            RocalIntParam mirror = NULL, RocalTensorLayout output_layout = ROCAL_NONE,
                                                            RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :1045
extern "C" RocalTensor ROCAL_API_CALL rocalRandomCrop(RocalContext context, RocalTensor input, bool is_output, RocalFloatParam crop_area_factor = NULL,
                                                      RocalFloatParam crop_aspect_ratio = NULL, RocalFloatParam crop_pos_x = NULL,
                                                      RocalFloatParam crop_pos_y = NULL, int num_of_attempts = 20,
                                                      RocalTensorLayout output_layout = ROCAL_NONE, RocalTensorOutputType output_datatype = ROCAL_UINT8);  // :1066

#endif  // ROCAL_API_MI355X_H
