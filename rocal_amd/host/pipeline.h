// Tensor / Graph / Node / pipeline context of the hot path, with rocAL's interface
// (rocAL/include/pipeline/tensor.h:65-309, graph.h:29-44, node.h:30-63, master_graph.h:245-263) on top of
// the C ABI in include/rocal_mi355x.h. A Node owns one rmx_op; Graph::process() launches the nodes in
// creation order on one stream (vxProcessGraph of the reference, rocAL/source/pipeline/graph.cpp:96-103) and
// records an event behind them; the wait for that event is where a consumer takes an output (MasterGraph::wait_outputs).
#pragma once
#include <cstdint>
#include <list>
#include <memory>
#include <string>
#include <vector>

#include "exception.h"
#include "rocal_api_mi355x.h"
#include "rocal_mi355x.h"

// rocAL/include/pipeline/commons.h:45-70,110-113 (same numeric values as the C ABI's enums)
enum class RocalTensorlayout { NHWC = 0, NCHW = 1, NONE = 9 };
enum class RocalTensorDataType { FP32 = 0, FP16 = 1, UINT8 = 2 };
enum class RocalROIType { LTRB = 0, XYWH = 1 };

// rocAL/include/pipeline/commons.h:115-140
union Roi2DCords {
    struct { unsigned l, t, r, b; } ltrb;
    struct { unsigned x, y, w, h; } xywh;
};

#include "packed_buffer.h"

class TensorInfo {
   public:
    TensorInfo() = default;
    // dims in the order of the layout: NHWC -> {N,H,W,C}, NCHW -> {N,C,H,W}
    TensorInfo(std::vector<size_t> dims, RocalTensorlayout layout, RocalTensorDataType dtype);
    size_t batch_size() const { return _dims.at(0); }
    const std::vector<size_t> &dims() const { return _dims; }
    RocalTensorlayout layout() const { return _layout; }
    RocalTensorDataType data_type() const { return _dtype; }
    RocalROIType roi_type() const { return _roi_type; }
    unsigned get_channels() const { return _channels; }
    // {max_width, max_height}, as TensorInfo::max_shape() for images (tensor.h:262)
    const std::vector<size_t> &max_shape() const { return _max_shape; }
    size_t data_size() const { return _data_size; }
    size_t data_type_size() const { return _dtype == RocalTensorDataType::FP32 ? 4 : _dtype == RocalTensorDataType::FP16 ? 2 : 1; }
    void set_data_type(RocalTensorDataType t) { _dtype = t; recompute(); }
    void set_roi_type(RocalROIType t) { _roi_type = t; }
    // Permutes the dims when the layout changes; the ROI buffer stays shared (tensor.h:205-214).
    void set_tensor_layout(RocalTensorlayout layout);
    // Changes the layout when `layout` is not NONE and sets the padded width/height (tensor.h:223-245).
    void modify_dims_width_and_height(RocalTensorlayout layout, size_t width, size_t height);
    Roi2DCords *roi() const { return _roi.get(); }
    void reallocate_roi() { _roi.reset(new Roi2DCords[batch_size()](), std::default_delete<Roi2DCords[]>()); reset_roi(); }
    void reset_roi();
    rmx_tensor_desc desc() const;

   private:
    void recompute();
    std::vector<size_t> _dims;
    RocalTensorlayout _layout = RocalTensorlayout::NHWC;
    RocalTensorDataType _dtype = RocalTensorDataType::UINT8;
    RocalROIType _roi_type = RocalROIType::XYWH;
    unsigned _channels = 3;
    std::vector<size_t> _max_shape{0, 0};
    size_t _data_size = 0;
    // Shared between copies of an info and re-allocated only when the padded width/height change
    // (tensor.h:203,248): the output of a node that keeps the size (colour ops, flip) aliases its input's ROI.
    std::shared_ptr<Roi2DCords> _roi;
};

class MasterGraph;

// rocAL/include/pipeline/tensor.h:316-388: the tensor behind the public rocalTensor interface.
class Tensor : public rocalTensor {
   public:
    explicit Tensor(const TensorInfo &info, MasterGraph *owner = nullptr) : _info(info), _owner(owner) {}
    const TensorInfo &info() const { return _info; }
    // the device address as the graph sees it (no wait): nodes, launches, bindings
    void *handle() const { return _buffer; }
    // ---- rocalTensor (what a consumer calls: buffer() and the copies wait for the batch that is being computed)
    void *buffer() override;
    unsigned copy_data(void *user_buffer, RocalOutputMemType external_mem_type) override;
    unsigned copy_data(void *user_buffer, unsigned int x_offset, unsigned int y_offset, unsigned int max_cols, unsigned int max_rows) override;
    unsigned num_of_dims() override { return (unsigned)_info.dims().size(); }
    unsigned batch_size() override { return (unsigned)_info.batch_size(); }
    std::vector<size_t> dims() override { return _info.dims(); }
    std::vector<size_t> strides() override;
    RocalTensorLayout layout() override { return (RocalTensorLayout)_info.layout(); }
    RocalTensorBackend backend() override { return ROCAL_GPU; }
    RocalTensorOutputType data_type() override { return (RocalTensorOutputType)_info.data_type(); }
    RocalOutputMemType mem_type() override { return ROCAL_MEMCPY_GPU; }
    size_t data_size() override { return _info.data_size(); }
    RocalROICordsType roi_type() override { return (RocalROICordsType)_info.roi_type(); }
    size_t get_roi_dims_size() override { return 2; }
    void copy_roi(void *roi_buffer) override;
    std::vector<size_t> shape() override { return _info.max_shape(); }
    void set_dims(std::vector<size_t>) override { THROW("the dimensions of a pipeline tensor are fixed by the node that produces it") }
    void set_mem_handle(void *buffer) override;
    void set_tensor_layout(RocalTensorLayout) override { THROW("the layout of a pipeline tensor is fixed by the node that produces it") }
    uint64_t data_type_size() override { return _info.data_type_size(); }
    // The loader / ring buffer hands a new device buffer every batch (tensor.cpp:478-489).
    void swap_handle(void *device_ptr) { _buffer = device_ptr; }
    // Clamps to the padded maxima like Tensor::update_tensor_roi (tensor.cpp:193-220).
    void update_tensor_roi(const std::vector<uint32_t> &width, const std::vector<uint32_t> &height);
    bool is_output = false;
    bool elided = false;  // virtual tensor inside a fused chain: never materialised
    // A source whose batch lies packed in its buffer (PackedCircularBuffer): the layout of the current batch, or null for
    // the dense [N, Hmax, Wmax, C] tensor. Nodes that read such a tensor hand the layout to their kernels before every update.
    const PackedLayout *ragged() const { return _ragged; }
    void set_ragged(const PackedLayout *l) { _ragged = l; }

   private:
    TensorInfo _info;
    MasterGraph *_owner = nullptr;
    void *_buffer = nullptr;
    const PackedLayout *_ragged = nullptr;
};

// rocAL/include/pipeline/tensor.h:391-422
class TensorList : public rocalTensorList {
   public:
    uint64_t size() override { return _tensor_list.size(); }
    Tensor *at(size_t index) override { return _tensor_list.at(index); }
    void push_back(Tensor *t) { _tensor_list.push_back(t); }
    void clear() { _tensor_list.clear(); }

   private:
    std::vector<Tensor *> _tensor_list;
};

class Node;

class Graph {
   public:
    enum class Status { OK = 0 };
    explicit Graph(int gpu_id, void *stream = nullptr);
    ~Graph();
    Status verify();
    Status process();  // enqueues the launches of every node; does not wait
    Status release();
    rmx_ctx *get() { return _ctx; }
    void add(Node *n) { _order.push_back(n); }
    // bilinear resize nodes clamp the right / lower neighbour at the last-but-one pixel of the window, as the reference's
    // device kernel does (rocAL/rocAL_hip/rocal_hip_kernels.cpp:339-345), instead of at the last pixel
    bool edge_device_rule = false;

   private:
    rmx_ctx *_ctx = nullptr;
    std::vector<Node *> _order;
};

class Node {
   public:
    Node(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs)
        : _inputs(inputs), _outputs(outputs), _batch_size(outputs[0]->info().batch_size()) {}
    virtual ~Node();
    void create(std::shared_ptr<Graph> graph);
    void update_parameters();
    std::vector<Tensor *> input() { return _inputs; }
    std::vector<Tensor *> output() { return _outputs; }
    void release();
    const Roi2DCords *get_src_roi() { return _inputs[0]->info().roi(); }
    const Roi2DCords *get_dst_roi() { return _outputs[0]->info().roi(); }
    // --- used by Graph ---
    virtual void launch();
    bool fused_away = false;  // this node's work is done by the launch of the node that precedes it
    // A CropMirrorNormalize node directly behind a resize node: the pair runs as one kernel.
    virtual bool try_absorb(Node *) { return false; }
    // A colour node and a CropMirrorNormalize node directly behind a bilinear resize node: the three run as one kernel.
    virtual bool try_absorb_chain(Node *, Node *) { return false; }
    // A colour node that can be the middle of such a chain says which stage it is (RMX_F_COLOR_LINEAR / RMX_F_COLOR_TWIST, 0 = none)
    // and, per batch, renews its parameters and hands out their arrays (NULL = neutral value).
    virtual unsigned chain_colour_kind() const { return 0; }
    virtual void chain_colour_refresh(const float *arrays[4]) { arrays[0] = arrays[1] = arrays[2] = arrays[3] = nullptr; }

   protected:
    virtual void create_node() = 0;
    virtual void update_node() = 0;
    const std::vector<Tensor *> _inputs;
    const std::vector<Tensor *> _outputs;
    std::shared_ptr<Graph> _graph = nullptr;
    rmx_op *_node = nullptr;
    size_t _batch_size;
    bool _ragged_source = false;  // the op currently reads a packed source
    void check(int status, const char *what);
    std::vector<uint32_t> roi_as_array(const Roi2DCords *roi) const;
};

// The part of Context + MasterGraph the hot path needs (rocAL/include/pipeline/master_graph.h:245-263,
// source/pipeline/master_graph.cpp:247-260,323-335,408,1010-1017): owns tensors and nodes, builds them
// on verify, and per batch renews parameters, updates every node and processes the graph.
class BoundingBoxGraph;
class MetaDataBatch;

class MasterGraph {
   public:
    MasterGraph(size_t batch_size, int gpu_id, void *stream);
    ~MasterGraph();
    Tensor *create_tensor(const TensorInfo &info, bool is_output);
    template <typename T>
    std::shared_ptr<T> add_node(const std::vector<Tensor *> &inputs, const std::vector<Tensor *> &outputs) {
        auto node = std::make_shared<T>(inputs, outputs);
        _nodes.push_back(node);
        return node;
    }
    void build();
    // One batch: parameters renewed, nodes updated, launches enqueued, an event recorded behind them. Does not wait.
    void run();
    // Blocks until the batch of the last run() is complete (the consumer side of the reference's output ring buffer:
    // ring_buffer.cpp:118-119 block_if_empty, called from get_output_tensors / copy_output, master_graph.cpp:859-938).
    void wait_outputs();
    void outputs_wait_on_stream(void *stream);
    TensorList *get_output_tensors();                        // master_graph.cpp:929-938
    void copy_output(unsigned char *out_ptr, size_t bytes);  // master_graph.cpp:859-927
    void stop_sources();                                     // wakes every thread blocked on a packed source
    void set_edge_rule(bool device_rule);
    bool edge_rule() const { return _graph->edge_device_rule; }
    void *stream() const;
    void set_output(Tensor *t);  // master_graph.cpp:337-349
    // A source tensor fed through a ring of packed batches (stands where the loader module and its CircularBuffer stand,
    // master_graph.cpp:1116-1160 / image_loader.cpp:115-170): run() takes the oldest batch of every such source.
    Tensor *create_packed_source(const TensorInfo &info, bool is_output, size_t slot_bytes, size_t depth);
    PackedCircularBuffer *packed_buffer(Tensor *source);
    // master_graph.cpp:514-856: converts the single u8 output tensor into a float tensor in caller memory
    void to_tensor(void *out_ptr, RocalTensorlayout format, float multiplier0, float multiplier1, float multiplier2, float offset0, float offset1,
                   float offset2, bool reverse_channels, RocalTensorDataType output_data_type, unsigned max_roi_height, unsigned max_roi_width);
    // bounding boxes that follow the images (master_graph.cpp:1004-1013): switched on before nodes are added,
    // a batch of boxes is handed in before each run and the transformed batch is read back after it
    void enable_meta_data();
    bool meta_data_enabled() const { return (bool)_meta_graph; }
    std::shared_ptr<BoundingBoxGraph> meta_graph() { return _meta_graph; }
    void set_input_meta_data(std::shared_ptr<MetaDataBatch> m) { _input_meta = m; }
    std::shared_ptr<MetaDataBatch> output_meta_data() { return _output_meta; }
    size_t batch_size() const { return _batch_size; }
    // Accumulated microseconds since the last call, which resets them (TimingDbg::get_timing, include/pipeline/timing_debug.h:72-82):
    // [0] parameter renewal + node updates, [1] Graph::process (master_graph.cpp:1015-1017), [2] to_tensor.
    void take_timing(unsigned long long out[3]);
    void give_back_timing(unsigned long long process_us, unsigned long long convert_us) {
        _time_us[1] += (double)process_us;
        _time_us[2] += (double)convert_us;
    }
    // an output tensor written straight into caller-owned device memory (Tensor::swap_handle, tensor.cpp:478-489)
    void bind_output(Tensor *t, void *device_ptr);
    const std::vector<Tensor *> &outputs() const { return _outputs; }
    bool built() const { return _built; }

   private:
    size_t _batch_size;
    int _gpu_id;
    std::shared_ptr<Graph> _graph;
    std::list<std::shared_ptr<Node>> _nodes;
    std::list<std::unique_ptr<Tensor>> _tensors;
    std::vector<Tensor *> _outputs;
    std::vector<void *> _owned_buffers;
    std::shared_ptr<BoundingBoxGraph> _meta_graph;
    std::shared_ptr<MetaDataBatch> _input_meta, _output_meta;
    bool _built = false;
    void *_done = nullptr;   // hipEvent_t behind the launches of the last run()
    bool _pending = false;   // a run() has been enqueued and nobody has waited for it yet
    TensorList _output_list;
    std::vector<std::pair<Tensor *, std::unique_ptr<PackedCircularBuffer>>> _packed_sources;
    double _time_us[3] = {0.0, 0.0, 0.0};
    // the conversion op of to_tensor(), rebuilt when the requested format changes
    rmx_op *_to_tensor_op = nullptr;
    unsigned _to_tensor_key[4] = {0, 0, 0, 0};
};

struct Context {
    Context(size_t batch_size, int gpu_id, void *stream) : master_graph(new MasterGraph(batch_size, gpu_id, stream)) {}
    std::unique_ptr<MasterGraph> master_graph;
    std::string error;
    unsigned long long update_time_us = 0;  // parameter-update time read off by rocalGetTimingInfo, kept for rocalGetParameterUpdateTime
    void capture_error(const std::string &e) { error = e; }
};
