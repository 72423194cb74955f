#include "pipeline.h"

#include <chrono>

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <iostream>

#include "meta.h"
#include "parameters.h"

/* ---------------------------------------------------------------- TensorInfo / Tensor */

TensorInfo::TensorInfo(std::vector<size_t> dims, RocalTensorlayout layout, RocalTensorDataType dtype)
    : _dims(std::move(dims)), _layout(layout), _dtype(dtype) {
    if (_dims.size() != 4) THROW("image tensors have 4 dimensions")
    recompute();
    reallocate_roi();
}

void TensorInfo::recompute() {
    if (_dims.size() != 4) return;
    if (_layout == RocalTensorlayout::NHWC) {
        _max_shape = {_dims[2], _dims[1]};
        _channels = (unsigned)_dims[3];
    } else {
        _max_shape = {_dims[3], _dims[2]};
        _channels = (unsigned)_dims[1];
    }
    _data_size = _dims[0] * _dims[1] * _dims[2] * _dims[3] * data_type_size();
}

void TensorInfo::modify_dims_width_and_height(RocalTensorlayout layout, size_t width, size_t height) {
    const size_t n = _dims[0], c = _channels;
    if (layout != RocalTensorlayout::NONE) _layout = layout;
    if (_layout == RocalTensorlayout::NHWC)
        _dims = {n, height, width, c};
    else
        _dims = {n, c, height, width};
    recompute();
    reallocate_roi();
}

void TensorInfo::set_tensor_layout(RocalTensorlayout layout) {
    if (layout == RocalTensorlayout::NONE || layout == _layout) return;
    const size_t n = _dims[0], c = _channels, w = _max_shape[0], h = _max_shape[1];
    _layout = layout;
    if (_layout == RocalTensorlayout::NHWC)
        _dims = {n, h, w, c};
    else
        _dims = {n, c, h, w};
    recompute();
}

void TensorInfo::reset_roi() {
    for (size_t i = 0; i < batch_size(); i++) {
        _roi.get()[i].xywh.x = 0;
        _roi.get()[i].xywh.y = 0;
        _roi.get()[i].xywh.w = (unsigned)_max_shape[0];
        _roi.get()[i].xywh.h = (unsigned)_max_shape[1];
    }
}

rmx_tensor_desc TensorInfo::desc() const {
    rmx_tensor_desc d;
    d.n = (uint32_t)_dims[0];
    d.w = (uint32_t)_max_shape[0];
    d.h = (uint32_t)_max_shape[1];
    d.c = _channels;
    d.layout = (int32_t)_layout;
    d.dtype = (int32_t)_dtype;
    return d;
}

void Tensor::update_tensor_roi(const std::vector<uint32_t> &width, const std::vector<uint32_t> &height) {
    const unsigned max_w = (unsigned)_info.max_shape()[0], max_h = (unsigned)_info.max_shape()[1];
    if (width.size() != height.size()) THROW("Batch size of Tensor height and width info does not match")
    if (width.size() != _info.batch_size())
        THROW("The batch size of actual Tensor height and width different from Tensor batch size " + TOSTR(width.size()) + " != " + TOSTR(_info.batch_size()))
    Roi2DCords *roi = _info.roi();
    for (size_t i = 0; i < width.size(); i++) {
        roi[i].xywh.w = std::min(width[i], max_w);
        roi[i].xywh.h = std::min(height[i], max_h);
    }
}

void *Tensor::buffer() {
    if (_owner) _owner->wait_outputs();
    return _buffer;
}

std::vector<size_t> Tensor::strides() {
    const std::vector<size_t> &d = _info.dims();
    std::vector<size_t> s(d.size(), _info.data_type_size());
    for (int i = (int)d.size() - 2; i >= 0; i--) s[i] = s[i + 1] * d[i + 1];
    return s;
}

// tensor.cpp:419-454
unsigned Tensor::copy_data(void *user_buffer, RocalOutputMemType external_mem_type) {
    if (!_buffer) return 0;
    if (!user_buffer) THROW("copy_data: null destination")
    if (_owner) _owner->wait_outputs();
    hipMemcpyKind kind;
    if (external_mem_type == ROCAL_MEMCPY_GPU) kind = hipMemcpyDeviceToDevice;
    else if (external_mem_type == ROCAL_MEMCPY_HOST || external_mem_type == ROCAL_MEMCPY_PINNED) kind = hipMemcpyDeviceToHost;
    else THROW("copy_data requested mem type not supported")
    hipError_t e = hipMemcpy(user_buffer, _buffer, _info.data_size(), kind);
    if (e != hipSuccess) THROW(std::string("copy_data::hipMemcpy failed: ") + hipGetErrorName(e))
    return 0;
}

// tensor.cpp:456-476: per sample, max_rows rows of max_cols elements from (x_offset, y_offset) of the sample's first
// plane (rows of max_shape[0] elements), densely packed into host memory. One 2-D copy per sample.
unsigned Tensor::copy_data(void *user_buffer, unsigned int x_offset, unsigned int y_offset, unsigned int max_cols, unsigned int max_rows) {
    if (!_buffer) return 0;
    if (!user_buffer) THROW("copy_data: null destination")
    if (_owner) _owner->wait_outputs();
    const size_t es = _info.data_type_size(), w = _info.max_shape()[0], h = _info.max_shape()[1];
    const size_t row_elems = _info.layout() == RocalTensorlayout::NHWC ? w * _info.get_channels() : w;
    if ((size_t)x_offset + max_cols > row_elems || (size_t)y_offset + max_rows > h) THROW("copy_data: the window exceeds the tensor")
    const size_t sample_bytes = _info.data_size() / _info.batch_size();
    for (size_t i = 0; i < _info.batch_size(); i++) {
        const unsigned char *src = static_cast<const unsigned char *>(_buffer) + i * sample_bytes + ((size_t)y_offset * row_elems + x_offset) * es;
        unsigned char *dst = static_cast<unsigned char *>(user_buffer) + i * (size_t)max_rows * max_cols * es;
        hipError_t e = hipMemcpy2D(dst, (size_t)max_cols * es, src, row_elems * es, (size_t)max_cols * es, max_rows, hipMemcpyDeviceToHost);
        if (e != hipSuccess) THROW(std::string("copy_data::hipMemcpy2D failed: ") + hipGetErrorName(e))
    }
    return 0;
}

void Tensor::copy_roi(void *roi_buffer) {
    if (!roi_buffer) THROW("copy_roi: null destination")
    memcpy(roi_buffer, _info.roi(), sizeof(Roi2DCords) * _info.batch_size());
}

void Tensor::set_mem_handle(void *buffer) {
    if (!buffer) THROW("Invalid buffer pointer passed")
    if (_owner) _owner->bind_output(this, buffer);
    else _buffer = buffer;
}

/* ---------------------------------------------------------------- Graph */

Graph::Graph(int gpu_id, void *stream) {
    if (rmx_ctx_create(gpu_id, stream, stream ? 0 : 1, &_ctx) != RMX_OK) THROW(std::string("rmx_ctx_create failed: ") + rmx_last_error())
}

Graph::~Graph() { release(); }

// Chain planning: a node may take over the work of the node that follows it (resize -> CropMirrorNormalize
// through a virtual tensor nobody else reads). Everything else about verification happens in rmx_create_*.
Graph::Status Graph::verify() {
    auto readers = [&](Tensor *t) {
        int n = 0;
        for (Node *k : _order)
            for (Tensor *in : k->input()) n += (in == t);
        return n;
    };
    // resize -> colour node -> CropMirrorNormalize through two virtual tensors nobody else reads
    for (size_t i = 0; i + 2 < _order.size(); i++) {
        Node *a = _order[i], *b = _order[i + 1], *c = _order[i + 2];
        if (a->fused_away || b->fused_away || c->fused_away) continue;
        Tensor *mid1 = a->output()[0], *mid2 = b->output()[0];
        if (b->input().size() != 1 || b->input()[0] != mid1 || c->input()[0] != mid2 || mid1->is_output || mid2->is_output) continue;
        if (readers(mid1) != 1 || readers(mid2) != 1) continue;
        if (a->try_absorb_chain(b, c)) {
            b->fused_away = c->fused_away = true;
            mid1->elided = mid2->elided = true;
        }
    }
    for (size_t i = 0; i + 1 < _order.size(); i++) {
        Node *a = _order[i], *b = _order[i + 1];
        if (a->fused_away || b->fused_away) continue;
        Tensor *mid = a->output()[0];
        if (b->input().size() != 1 || b->input()[0] != mid || mid->is_output) continue;
        if (readers(mid) != 1) continue;  // counts every input of every node: a two-input node may read it as its second
        if (a->try_absorb(b)) {
            b->fused_away = true;
            mid->elided = true;
        }
    }
    return Status::OK;
}

Graph::Status Graph::process() {
    for (Node *n : _order)
        if (!n->fused_away) n->launch();
    return Status::OK;
}

Graph::Status Graph::release() {
    if (_ctx) {
        rmx_ctx_destroy(_ctx);
        _ctx = nullptr;
    }
    return Status::OK;
}

/* ---------------------------------------------------------------- Node */

Node::~Node() { release(); }

void Node::create(std::shared_ptr<Graph> graph) {
    if (_outputs.empty() || _inputs.empty()) THROW("Uninitialized input/output arguments")
    _graph = graph;
    create_node();  // a node that is fused away still sets up its parameters here, on the user thread
}

void Node::update_parameters() {
    // a packed source batch: its layout goes to the kernels before the node's own update (which clips the windows to each image)
    if (_node && !_inputs.empty()) {
        const PackedLayout *l = _inputs[0]->ragged();
        if (l) {
            check(rmx_op_set_ragged_source_strided(_node, l->offsets.data(), l->widths.data(), l->heights.data(), l->row_strides.data(), l->bytes),
                  "rmx_op_set_ragged_source_strided");
            _ragged_source = true;
        } else if (_ragged_source) {
            check(rmx_op_set_ragged_source(_node, nullptr, nullptr, nullptr, 0), "rmx_op_set_ragged_source");
            _ragged_source = false;
        }
    }
    update_node();
}

void Node::release() {
    if (_node) {
        rmx_op_destroy(_node);
        _node = nullptr;
    }
}

void Node::launch() {
    Tensor *in = _inputs[0], *out = _outputs[0];
    if (!in->handle() || !out->handle()) THROW("tensor without a device buffer at launch")
    check(rmx_op_launch(_node, in->handle(), out->handle()), "rmx_op_launch");
}

void Node::check(int status, const char *what) {
    if (status != RMX_OK) THROW(std::string(what) + " failed: " + rmx_last_error())
}

std::vector<uint32_t> Node::roi_as_array(const Roi2DCords *roi) const {
    std::vector<uint32_t> out(4 * _batch_size);
    for (size_t i = 0; i < _batch_size; i++) {
        out[4 * i + 0] = roi[i].xywh.x;
        out[4 * i + 1] = roi[i].xywh.y;
        out[4 * i + 2] = roi[i].xywh.w;
        out[4 * i + 3] = roi[i].xywh.h;
    }
    return out;
}

/* ---------------------------------------------------------------- MasterGraph */

MasterGraph::MasterGraph(size_t batch_size, int gpu_id, void *stream) : _batch_size(batch_size), _gpu_id(gpu_id), _graph(std::make_shared<Graph>(gpu_id, stream)) {
    hipEvent_t e;
    if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) THROW("hipEventCreate failed")
    _done = e;
    const char *edge = getenv("ROCAL_BILINEAR_EDGE");
    _graph->edge_device_rule = edge && (!strcmp(edge, "1") || !strcmp(edge, "device"));
}

MasterGraph::~MasterGraph() {
    // loader threads blocked on a packed source leave with an exception before anything they use is freed
    stop_sources();
    _packed_sources.clear();
    try {
        wait_outputs();
    } catch (...) {
    }
    if (_done) (void)hipEventDestroy(static_cast<hipEvent_t>(_done));
    if (_to_tensor_op) rmx_op_destroy(_to_tensor_op);
    _nodes.clear();
    for (void *p : _owned_buffers) (void)hipFree(p);
}

Tensor *MasterGraph::create_tensor(const TensorInfo &info, bool is_output) {
    _tensors.emplace_back(new Tensor(info, this));
    Tensor *t = _tensors.back().get();
    t->is_output = is_output;
    if (is_output) _outputs.push_back(t);
    return t;
}

// rocalVerify: plan chains, create every node's op on the user thread, then give every tensor that is
// written by a launch a device buffer (the reference's ring buffer / virtual tensors).
void MasterGraph::set_output(Tensor *t) {
    if (!t) THROW("null output tensor")
    if (_built) THROW("outputs must be set before rocalVerify")
    if (t->is_output) return;
    t->is_output = true;
    _outputs.push_back(t);
}

void MasterGraph::build() {
    if (_built) THROW("graph already built")
    for (auto &n : _nodes) _graph->add(n.get());
    _graph->verify();
    for (auto &n : _nodes) n->create(_graph);
    for (auto &n : _nodes) {
        Tensor *out = n->output()[0];
        if (out->elided || out->handle()) continue;
        void *p = nullptr;
        if (hipMalloc(&p, out->info().data_size() + 64) != hipSuccess) THROW("hipMalloc of " + TOSTR(out->info().data_size()) + " bytes failed")
        if (hipMemset(p, 0, out->info().data_size() + 64) != hipSuccess) THROW("hipMemset failed")
        _owned_buffers.push_back(p);
        out->swap_handle(p);
    }
    _built = true;
}

// One batch: master_graph.cpp:408 (renew), :1010-1013 (update_parameters per node), :1015-1017 (process).
namespace {
struct StopWatch {
    explicit StopWatch(double &acc) : _acc(acc), _t0(std::chrono::high_resolution_clock::now()) {}
    ~StopWatch() { _acc += std::chrono::duration<double, std::micro>(std::chrono::high_resolution_clock::now() - _t0).count(); }
    double &_acc;
    std::chrono::high_resolution_clock::time_point _t0;
};
}  // namespace

void MasterGraph::take_timing(unsigned long long out[3]) {
    for (int i = 0; i < 3; i++) {
        out[i] = (unsigned long long)_time_us[i];
        _time_us[i] = 0.0;
    }
}

void MasterGraph::bind_output(Tensor *t, void *device_ptr) {
    if (!t || !device_ptr) THROW("null tensor or buffer")
    if (((uintptr_t)device_ptr & 15u) != 0) THROW("an output buffer must be 16-byte aligned")
    if (t->elided) THROW("the tensor was fused away: it is never written")
    bool produced = false;
    for (auto &n : _nodes) produced = produced || (!n->output().empty() && n->output()[0] == t);
    if (!produced) THROW("the tensor is not the output of a node of this context")
    t->swap_handle(device_ptr);
}

Tensor *MasterGraph::create_packed_source(const TensorInfo &info, bool is_output, size_t slot_bytes, size_t depth) {
    Tensor *t = create_tensor(info, is_output);
    std::unique_ptr<PackedCircularBuffer> buf(new PackedCircularBuffer(_gpu_id, rmx_ctx_stream(_graph->get())));
    buf->init(_batch_size, slot_bytes, depth);
    _packed_sources.emplace_back(t, std::move(buf));
    return t;
}

PackedCircularBuffer *MasterGraph::packed_buffer(Tensor *source) {
    for (auto &p : _packed_sources)
        if (p.first == source) return p.second.get();
    THROW("the tensor is not a packed source")
}

void MasterGraph::run() {
    if (!_built) THROW("rocalVerify must be called before rocalRun")
    // the oldest batch of every packed source: its device slot becomes the tensor's buffer (the graph's stream waits for
    // the slot's copy), its layout and image sizes the tensor's (loader_module->load_next, master_graph.cpp:1134-1147)
    for (auto &p : _packed_sources) {
        if (p.second->level() == 0) THROW("rocalRun: a packed source has no batch (push one first)")
        p.first->swap_handle(p.second->get_read_buffer_dev());
        const PackedLayout &l = p.second->get_read_layout();
        p.first->set_ragged(&l);
        p.first->update_tensor_roi(l.widths, l.heights);
    }
    struct PopAtExit {  // the slots are given back when the launches are enqueued, also when a node throws
        std::vector<std::pair<Tensor *, std::unique_ptr<PackedCircularBuffer>>> &v;
        ~PopAtExit() {
            for (auto &p : v) {
                try {
                    p.second->pop();
                } catch (...) {
                }
            }
        }
    } pop_at_exit{_packed_sources};
    {
        StopWatch w(_time_us[0]);
        ParameterFactory::instance()->renew_parameters();
        for (auto &n : _nodes) n->update_parameters();
    }
    if (_meta_graph && _input_meta) {
        if (_input_meta->size() != _batch_size) THROW("bounding boxes were given for " + TOSTR(_input_meta->size()) + " samples, the batch has " + TOSTR(_batch_size))
        // an empty instance when nodes will fill it, a copy when no node touches the boxes
        _output_meta = _input_meta->clone(_meta_graph->_meta_nodes.empty());
        _meta_graph->process(_input_meta, _output_meta);
    }
    StopWatch w(_time_us[1]);
    _graph->process();
    if (hipEventRecord(static_cast<hipEvent_t>(_done), static_cast<hipStream_t>(stream())) != hipSuccess) THROW("hipEventRecord failed")
    _pending = true;
}

void *MasterGraph::stream() const { return rmx_ctx_stream(_graph->get()); }

// The wait counts as process time, which in the reference brackets the (synchronous) vxProcessGraph: master_graph.cpp:1015-1017.
void MasterGraph::wait_outputs() {
    if (!_pending) return;
    StopWatch w(_time_us[1]);
    _pending = false;
    const hipError_t e = hipEventSynchronize(static_cast<hipEvent_t>(_done));
    if (e != hipSuccess) THROW(std::string("waiting for the batch failed: ") + hipGetErrorString(e))
}

void MasterGraph::outputs_wait_on_stream(void *stream) {
    if (!_pending) return;
    if (hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(_done), 0) != hipSuccess) THROW("hipStreamWaitEvent failed")
}

TensorList *MasterGraph::get_output_tensors() {
    if (!_built) THROW("rocalVerify must be called before rocalGetOutputTensors")
    wait_outputs();
    _output_list.clear();
    for (Tensor *t : _outputs) _output_list.push_back(t);
    return &_output_list;
}

void MasterGraph::copy_output(unsigned char *out_ptr, size_t bytes) {
    if (!_built) THROW("rocalVerify must be called before rocalCopyToOutput")
    if (_outputs.size() != 1) THROW("Cannot copy, Multiple output tensors present in the list")
    if (!out_ptr) THROW("rocalCopyToOutput needs an output pointer")
    if (bytes != _outputs[0]->info().data_size()) THROW("rocalCopyToOutput: out_size " + TOSTR(bytes) + " is not the output's " + TOSTR(_outputs[0]->info().data_size()) + " bytes")
    StopWatch w(_time_us[2]);
    _outputs[0]->copy_data(out_ptr, ROCAL_MEMCPY_HOST);
}

void MasterGraph::stop_sources() {
    for (auto &p : _packed_sources) p.second->stop();
}

void MasterGraph::set_edge_rule(bool device_rule) {
    if (!_nodes.empty()) THROW("the bilinear edge rule must be chosen before the first node is added")
    _graph->edge_device_rule = device_rule;
}

void MasterGraph::enable_meta_data() {
    if (!_nodes.empty()) THROW("bounding boxes must be switched on before the first augmentation is added")
    if (!_meta_graph) _meta_graph = std::make_shared<BoundingBoxGraph>();
}

// master_graph.cpp:514-535 (checks) and :612-632 (device branch). The reference walks the read buffers of its
// ring and launches Hip_CopyInt8ToNHWC/NCHW once per buffer; here the output tensor is one buffer and the
// conversion is one launch of the library's ToTensor op on the graph's stream, followed by a wait, so that
// out_ptr is complete when the call returns.
void MasterGraph::to_tensor(void *out_ptr, RocalTensorlayout format, float multiplier0, float multiplier1, float multiplier2, float offset0,
                            float offset1, float offset2, bool reverse_channels, RocalTensorDataType output_data_type, unsigned max_roi_height,
                            unsigned max_roi_width) {
    if (!_built) THROW("rocalVerify must be called before rocalToTensor")
    StopWatch w(_time_us[2]);
    if (_outputs.size() != 1) THROW("Cannot copy, Multiple output tensors present in the list")
    Tensor *src = _outputs[0];
    const TensorInfo &info = src->info();
    if (info.data_type() != RocalTensorDataType::UINT8) THROW("The output tensor is not of UINT8 type")
    if (info.layout() != RocalTensorlayout::NHWC) THROW("The output tensor is not interleaved RGB")
    if (!out_ptr) THROW("rocalToTensor needs a device output pointer")
    if (!src->handle()) THROW("The output tensor has no buffer yet")
    rmx_tensor_desc s = info.desc(), d = s;
    if (max_roi_height == 0 || max_roi_width == 0) {
        max_roi_height = s.h;
        max_roi_width = s.w;
    }
    if (max_roi_height > s.h || max_roi_width > s.w) THROW("max_roi_height/max_roi_width exceed the output tensor")
    d.h = max_roi_height;
    d.w = max_roi_width;
    d.layout = (int32_t)format;
    d.dtype = (int32_t)output_data_type;
    const unsigned key[4] = {(unsigned)d.layout, (unsigned)d.dtype, d.h, d.w};
    if (!_to_tensor_op || !std::equal(key, key + 4, _to_tensor_key)) {
        if (_to_tensor_op) rmx_op_destroy(_to_tensor_op);
        _to_tensor_op = nullptr;
        if (rmx_create_to_tensor(_graph->get(), &s, &d, &_to_tensor_op) != RMX_OK) THROW("rmx_create_to_tensor: " + std::string(rmx_last_error()))
        std::copy(key, key + 4, _to_tensor_key);
    }
    const float mul[3] = {multiplier0, multiplier1, multiplier2}, add[3] = {offset0, offset1, offset2};
    if (rmx_update_to_tensor(_to_tensor_op, mul, add, reverse_channels ? 1 : 0) != RMX_OK) THROW("rmx_update_to_tensor: " + std::string(rmx_last_error()))
    // (same stream as the batch's launches: the conversion runs behind them, and the wait below covers both)
    if (rmx_op_launch(_to_tensor_op, src->handle(), out_ptr) != RMX_OK) THROW("rmx_op_launch: " + std::string(rmx_last_error()))
    if (rmx_ctx_sync(_graph->get()) != RMX_OK) THROW("rmx_ctx_sync: " + std::string(rmx_last_error()))
    _pending = false;
}
