#include "packed_buffer.h"

#include <hip/hip_runtime_api.h>

#include <cstdlib>

#include "exception.h"

#define HIP_OK(call, what)                                                                        \
    do {                                                                                          \
        hipError_t e_ = (call);                                                                   \
        if (e_ != hipSuccess) THROW(std::string(what) + " failed: " + hipGetErrorString(e_))      \
    } while (0)

PackedCircularBuffer::PackedCircularBuffer(int device, void *consumer_stream) : _device(device), _consumer_stream(consumer_stream) {}

// Counts the calling thread into the ring for the length of a call that touches the slots, and refuses it once the ring
// is closing: release() frees the slots only when the count is back at 0.
struct PackedCircularBuffer::Inside {
    explicit Inside(PackedCircularBuffer &b) : _b(b) {
        std::unique_lock<std::mutex> lock(_b._lock);
        if (_b._closing) THROW("the packed batch buffer was released")
        _b._inside++;
    }
    ~Inside() {
        bool idle;
        {
            std::unique_lock<std::mutex> lock(_b._lock);
            idle = --_b._inside == 0;
        }
        if (idle) _b._idle.notify_all();
    }
    PackedCircularBuffer &_b;
};

PackedCircularBuffer::~PackedCircularBuffer() { release(); }

void PackedCircularBuffer::init(size_t batch_size, size_t slot_bytes, size_t buff_depth) {
    if (_initialized) return;
    if (batch_size == 0 || slot_bytes == 0) THROW("PackedCircularBuffer: batch size and slot size must be non-zero")
    if (buff_depth < 2) THROW("PackedCircularBuffer: a depth of at least 2 is needed (one slot is being read while one is written)")
    _batch_size = batch_size;
    _slot_bytes = (slot_bytes + 255) / 256 * 256;
    _buff_depth = buff_depth;
    for (size_t i = 0; _device < 0 && i < buff_depth; i++) {
        void *h = malloc(_slot_bytes);
        if (!h) THROW("out of host memory for a packed batch slot")
        _host_buffer_ptrs.push_back(static_cast<unsigned char *>(h));
        _dev_buffer.push_back(h);
        _copied.push_back(nullptr);
        _consumed.push_back(nullptr);
    }
    if (_device >= 0) {
        HIP_OK(hipSetDevice(_device), "hipSetDevice");
        hipStream_t s;
        HIP_OK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");
        _copy_stream = s;
    }
    for (size_t i = 0; _device >= 0 && i < buff_depth; i++) {
        void *h = nullptr, *d = nullptr;
        hipEvent_t a, b;
        // pinned memory is allocated, never registered; 16 spare bytes behind the slot keep the kernels' wide loads inside it
        HIP_OK(hipHostMalloc(&h, _slot_bytes, hipHostMallocDefault), "hipHostMalloc of a packed batch slot");
        HIP_OK(hipMalloc(&d, _slot_bytes + 16), "hipMalloc of a packed batch slot");
        HIP_OK(hipEventCreateWithFlags(&a, hipEventDisableTiming), "hipEventCreate");
        HIP_OK(hipEventCreateWithFlags(&b, hipEventDisableTiming), "hipEventCreate");
        _host_buffer_ptrs.push_back(static_cast<unsigned char *>(h));
        _dev_buffer.push_back(d);
        _copied.push_back(a);
        _consumed.push_back(b);
    }
    _layout.resize(buff_depth);
    for (auto &l : _layout) {
        l.offsets.assign(batch_size, 0);
        l.widths.assign(batch_size, 0);
        l.heights.assign(batch_size, 0);
        l.row_strides.assign(batch_size, 0);
    }
    _placed.assign(batch_size, false);
    _write_pos = 0;
    _closing = false;
    _initialized = true;
}

void PackedCircularBuffer::stop() {
    {
        std::unique_lock<std::mutex> lock(_lock);
        _closing = true;
    }
    _wait_for_load.notify_all();
    _wait_for_unload.notify_all();
}

bool PackedCircularBuffer::stopped() {
    std::unique_lock<std::mutex> lock(_lock);
    return _closing;
}

void PackedCircularBuffer::release() {
    if (!_initialized) return;
    stop();
    {
        // a loader thread that was blocked in place_image() leaves with an exception; the slots stay until it has left
        std::unique_lock<std::mutex> lock(_lock);
        _idle.wait(lock, [&] { return _inside == 0; });
    }
    if (_device < 0) {
        for (unsigned char *h : _host_buffer_ptrs) free(h);
        _host_buffer_ptrs.clear();
        _dev_buffer.clear();
        _copied.clear();
        _consumed.clear();
        _initialized = false;
        return;
    }
    (void)hipSetDevice(_device);
    (void)hipStreamSynchronize(static_cast<hipStream_t>(_copy_stream));
    for (size_t i = 0; i < _buff_depth; i++) {
        (void)hipEventSynchronize(static_cast<hipEvent_t>(_consumed[i]));
        (void)hipEventDestroy(static_cast<hipEvent_t>(_copied[i]));
        (void)hipEventDestroy(static_cast<hipEvent_t>(_consumed[i]));
        (void)hipHostFree(_host_buffer_ptrs[i]);
        (void)hipFree(_dev_buffer[i]);
    }
    (void)hipStreamDestroy(static_cast<hipStream_t>(_copy_stream));
    _host_buffer_ptrs.clear();
    _dev_buffer.clear();
    _copied.clear();
    _consumed.clear();
    _initialized = false;
}

unsigned char *PackedCircularBuffer::get_write_buffer() {
    if (!_initialized) THROW("Circular buffer not initialized")
    Inside in(*this);
    block_if_full();
    std::unique_lock<std::mutex> lock(_lock);
    // woken without room (stop() or unblock_writer()): the slot at the write pointer is still the reader's or the copy's
    if (_closing) THROW("the packed batch buffer was released")
    if (full()) THROW("the packed batch buffer is full (the writer was unblocked without a free slot)")
    return _host_buffer_ptrs[_write_ptr];
}

unsigned char *PackedCircularBuffer::place_image(size_t index, uint32_t width, uint32_t height, uint32_t *row_stride) {
    if (!_initialized) THROW("Circular buffer not initialized")
    if (index >= _batch_size) THROW("image index " + TOSTR(index) + " outside the batch of " + TOSTR(_batch_size))
    if (width == 0 || height == 0) THROW("image " + TOSTR(index) + " is empty")
    if (_placed[index]) THROW("image " + TOSTR(index) + " was placed twice in one batch")
    Inside in(*this);
    unsigned char *base = get_write_buffer();
    if (_write_pos == 0 && _device >= 0) {
        // first image of a batch: the copy that last read this pinned slot has finished (a consumer that does not wait for
        // its batches can be a whole ring behind the loader)
        HIP_OK(hipSetDevice(_device), "hipSetDevice");
        HIP_OK(hipEventSynchronize(static_cast<hipEvent_t>(_copied[_write_ptr])), "hipEventSynchronize");
    }
    const uint32_t stride = (width * 3u + 3u) / 4u * 4u;
    const uint64_t bytes = (uint64_t)stride * height;
    if (_write_pos + bytes > _slot_bytes)
        THROW("packed batch exceeds its slot: image " + TOSTR(index) + " needs " + TOSTR(bytes) + " bytes at " + TOSTR(_write_pos) + " of " + TOSTR(_slot_bytes))
    PackedLayout &l = _layout[_write_ptr];
    l.offsets[index] = _write_pos;
    l.widths[index] = width;
    l.heights[index] = height;
    l.row_strides[index] = stride;
    _placed[index] = true;
    unsigned char *p = base + _write_pos;
    _write_pos += bytes;
    if (row_stride) *row_stride = stride;
    return p;
}

void PackedCircularBuffer::push() {
    if (!_initialized) return;
    Inside in(*this);
    for (size_t i = 0; i < _batch_size; i++)
        if (!_placed[i]) THROW("push: image " + TOSTR(i) + " of the batch was not placed")
    PackedLayout &l = _layout[_write_ptr];
    l.bytes = _write_pos;
    if (_device >= 0) {
        HIP_OK(hipSetDevice(_device), "hipSetDevice");
        auto cs = static_cast<hipStream_t>(_copy_stream);
        // the kernels that read this device slot the last time round have finished before it is overwritten
        HIP_OK(hipStreamWaitEvent(cs, static_cast<hipEvent_t>(_consumed[_write_ptr]), 0), "hipStreamWaitEvent");
        HIP_OK(hipMemcpyAsync(_dev_buffer[_write_ptr], _host_buffer_ptrs[_write_ptr], l.bytes, hipMemcpyHostToDevice, cs), "hipMemcpyAsync of a packed batch");
        HIP_OK(hipEventRecord(static_cast<hipEvent_t>(_copied[_write_ptr]), cs), "hipEventRecord");
    }
    {
        std::unique_lock<std::mutex> lock(_names_buff_lock);
        _circ_buff_data_info.push(_last_data_info);
    }
    _placed.assign(_batch_size, false);
    _write_pos = 0;
    {
        std::unique_lock<std::mutex> lock(_lock);
        _write_ptr = (_write_ptr + 1) % _buff_depth;
        _level++;
    }
    _wait_for_load.notify_all();
}

void *PackedCircularBuffer::get_read_buffer_dev() {
    if (!_initialized) THROW("Circular buffer not initialized")
    Inside in(*this);
    block_if_empty();
    {
        std::unique_lock<std::mutex> lock(_lock);
        if (_closing) THROW("the packed batch buffer was released")
        if (empty()) THROW("the packed batch buffer is empty")  // (unblocked without a batch)
    }
    if (_device >= 0)
        HIP_OK(hipStreamWaitEvent(static_cast<hipStream_t>(_consumer_stream), static_cast<hipEvent_t>(_copied[_read_ptr]), 0), "hipStreamWaitEvent");
    return _dev_buffer[_read_ptr];
}

const PackedLayout &PackedCircularBuffer::get_read_layout() {
    if (!_initialized) THROW("Circular buffer not initialized")
    return _layout[_read_ptr];
}

DecodedDataInfo &PackedCircularBuffer::get_decoded_data_info() {
    std::unique_lock<std::mutex> lock(_names_buff_lock);
    if (_circ_buff_data_info.empty()) THROW("no batch information in the buffer")
    return _circ_buff_data_info.front();
}

void PackedCircularBuffer::pop() {
    if (!_initialized) return;
    Inside in(*this);
    if (level() == 0) THROW("pop on an empty packed batch buffer")
    // whatever has been enqueued on the consumer stream so far reads the slot: the writer's next copy into it waits for that
    if (_device >= 0)
        HIP_OK(hipEventRecord(static_cast<hipEvent_t>(_consumed[_read_ptr]), static_cast<hipStream_t>(_consumer_stream)), "hipEventRecord");
    {
        std::unique_lock<std::mutex> lock(_names_buff_lock);
        if (!_circ_buff_data_info.empty()) _circ_buff_data_info.pop();
    }
    {
        std::unique_lock<std::mutex> lock(_lock);
        _read_ptr = (_read_ptr + 1) % _buff_depth;
        _level--;
    }
    _wait_for_unload.notify_all();
}

size_t PackedCircularBuffer::level() {
    std::unique_lock<std::mutex> lock(_lock);
    return _level;
}

// Empties the ring for a new epoch (circular_buffer.cpp:333-343). Threads blocked on it are woken and turned away first,
// and the call waits until they have left; the ring then takes batches again.
void PackedCircularBuffer::reset() {
    stop();
    std::unique_lock<std::mutex> lock(_lock);
    _idle.wait(lock, [&] { return _inside == 0; });
    _write_ptr = _read_ptr = _level = 0;
    _write_pos = 0;
    _placed.assign(_batch_size, false);
    {
        std::unique_lock<std::mutex> names(_names_buff_lock);
        while (!_circ_buff_data_info.empty()) _circ_buff_data_info.pop();
    }
    _released_reader = _released_writer = false;
    _closing = false;
}

void PackedCircularBuffer::block_if_empty() {
    std::unique_lock<std::mutex> lock(_lock);
    _wait_for_load.wait(lock, [&] { return !empty() || _released_reader || _closing; });
    _released_reader = false;
}

void PackedCircularBuffer::block_if_full() {
    std::unique_lock<std::mutex> lock(_lock);
    _wait_for_unload.wait(lock, [&] { return !full() || _released_writer || _closing; });
    _released_writer = false;
}

void PackedCircularBuffer::unblock_reader() {
    {
        std::unique_lock<std::mutex> lock(_lock);
        _released_reader = true;
    }
    _wait_for_load.notify_all();
}

void PackedCircularBuffer::unblock_writer() {
    {
        std::unique_lock<std::mutex> lock(_lock);
        _released_writer = true;
    }
    _wait_for_unload.notify_all();
}
