// Loader -> device hand-off for ragged batches: a ring of packed batch buffers with the interface of rocAL's
// CircularBuffer (rocAL/include/loaders/circular_buffer.h:48-110, source/loaders/circular_buffer.cpp:65-160,299-343):
// the loader thread takes the write buffer, places the decoded images and pushes; the output thread takes the read
// buffer on the device and pops. Two things differ, on purpose:
//   * a slot holds the images of a batch one behind the other, every image and every row at a multiple of 4 bytes,
//     instead of a padded [N, Hmax, Wmax, 3] tensor (the reference pads: image_read_and_decode.cpp:165-390), with a layout
//     entry per image (offset, width, height, row stride) that the kernels read through rmx_op_set_ragged_source_strided;
//   * push() starts ONE asynchronous copy of the bytes that were written, on a copy stream of its own, where the
//     reference copies the whole padded slot with a blocking hipMemcpy (circular_buffer.cpp:118-123). A RandomResizedCrop
//     batch of 256 images up to 640 x 640 is 315 MB padded and about 80 MB packed.
#pragma once
#include <condition_variable>
#include <cstdint>
#include <mutex>
#include <queue>
#include <string>
#include <vector>

// Names and sizes of the images of a batch (circular_buffer.h:33-42, the members the image path uses).
struct DecodedDataInfo {
    std::vector<std::string> _data_names;
    std::vector<uint32_t> _roi_width, _roi_height;
    std::vector<uint32_t> _original_width, _original_height;
};

// Where the images of a packed batch lie.
struct PackedLayout {
    std::vector<uint64_t> offsets;
    std::vector<uint32_t> widths, heights, row_strides;
    uint64_t bytes = 0;  // used bytes of the slot
};

class PackedCircularBuffer {
   public:
    // consumer_stream: the stream the kernels that read the batches run on (hipStream_t as void *).
    // device < 0: a ring in plain host memory (the reference's RocalMemType::HOST): no device slots, no copies, no HIP call;
    // get_read_buffer_dev() then returns the host slot.
    PackedCircularBuffer(int device, void *consumer_stream);
    ~PackedCircularBuffer();
    // slot_bytes: capacity of a slot (packed bytes of the largest batch); buff_depth slots, one of which is the one being read
    void init(size_t batch_size, size_t slot_bytes, size_t buff_depth);
    // Shut-down, as the reference's loaders do it before they let go of their buffer (image_loader.cpp:84,126-127,241:
    // unblock_writer / unblock_reader): stop() wakes every thread blocked on the ring and turns it, and every later caller,
    // away with an exception ("released") instead of a slot; it is sticky until reset(). release() stops the ring, waits
    // until no thread is inside one of its calls any more and only then frees the slots.
    void stop();
    bool stopped();
    void release();
    // ---- writer side (loader thread)
    unsigned char *get_write_buffer();  // pinned host memory of the slot being filled; blocks the caller if the buffer is full
    // Reserves the place of image `index` in the slot being filled (images in any order, each once per batch) and returns
    // where its first row goes; rows are `row_stride` bytes apart (width * 3 rounded up to a multiple of 4).
    unsigned char *place_image(size_t index, uint32_t width, uint32_t height, uint32_t *row_stride);
    void set_decoded_data_info(const DecodedDataInfo &info) { _last_data_info = info; }
    void push();  // the slot is complete: starts its copy to the device and makes it available to the reader
    // ---- reader side (output thread)
    void *get_read_buffer_dev();              // blocks the caller if the buffer is empty; the consumer stream waits for the slot's copy
    const PackedLayout &get_read_layout();    // layout of the slot get_read_buffer_dev() returns
    DecodedDataInfo &get_decoded_data_info();
    void pop();  // the kernels that read the slot have been enqueued: the slot is free once they have run
    // ----
    size_t level();
    void reset();
    void block_if_empty();
    void block_if_full();
    void unblock_reader();
    void unblock_writer();
    size_t slot_bytes() const { return _slot_bytes; }

   private:
    bool full() const { return _level >= _buff_depth - 1; }  // the last spot is the one the reader holds (circular_buffer.cpp:303-305)
    bool empty() const { return _level == 0; }
    int _device;
    void *_consumer_stream;
    void *_copy_stream = nullptr;
    size_t _batch_size = 0, _slot_bytes = 0, _buff_depth = 0;
    std::vector<unsigned char *> _host_buffer_ptrs;
    std::vector<void *> _dev_buffer;
    std::vector<void *> _copied, _consumed;  // hipEvent_t per slot: copy finished / readers finished
    std::vector<PackedLayout> _layout;       // per slot
    std::vector<bool> _placed;               // images placed in the slot being filled
    uint64_t _write_pos = 0;
    DecodedDataInfo _last_data_info;
    std::queue<DecodedDataInfo> _circ_buff_data_info;
    std::mutex _lock, _names_buff_lock;
    std::condition_variable _wait_for_load, _wait_for_unload;
    size_t _write_ptr = 0, _read_ptr = 0, _level = 0;
    bool _initialized = false, _released_reader = false, _released_writer = false;
    bool _closing = false;           // stop() was called: nobody is handed a slot any more
    size_t _inside = 0;              // threads inside a call that touches the slots
    std::condition_variable _idle;   // signalled when _inside falls to 0
    struct Inside;                   // scope guard that counts a thread in and out
};
