"""Pipeline of the Python API (rocAL_pybind/amd/rocal/pipeline.py:66-170): owns the context, is the `with` scope in which the
fn.* calls add nodes, marks outputs, builds and runs. Readers and decoders are outside the hot path: a pipeline here takes
its decoded batches from device memory (device_source / feed)."""
from . import backend, types

b = backend.Backend()


class Pipeline:
    _current_pipeline = None

    def __init__(self, batch_size=-1, num_threads=0, device_id=0, seed=1, exec_pipelined=True, prefetch_queue_depth=2, exec_async=True,
                 bytes_per_sample=0, rocal_cpu=False, max_streams=-1, default_cuda_stream_priority=0, tensor_layout=types.NCHW,
                 reverse_channels=False, mean=None, std=None, tensor_dtype=types.FLOAT, output_memory_type=None):
        if rocal_cpu:
            raise Exception("Failed creating the pipeline: this build has no CPU path (rocal_cpu=True)")
        self._handle = b.rocalCreate(batch_size, types.GPU, device_id, num_threads, prefetch_queue_depth, tensor_dtype)
        if b.getStatus(self._handle) != types.OK:
            raise Exception("Failed creating the pipeline")
        self._batch_size = batch_size
        self._device_id = device_id
        self._seed = seed
        self._tensor_layout = tensor_layout
        self._tensor_dtype = tensor_dtype
        # pipeline.py:100-103: what copyToExternalTensor applies to a u8 output
        self._multiplier = list(map(lambda x: 1 / x, std)) if std else [1.0, 1.0, 1.0]
        self._offset = list(map(lambda x, y: -(x / y), mean, std)) if mean and std else [0.0, 0.0, 0.0]
        self._reverse_channels = reverse_channels
        self._output_memory_type = output_memory_type if output_memory_type else types.DEVICE_MEMORY
        self._outputs = []
        self.set_seed(self._seed)

    def __enter__(self):
        Pipeline._current_pipeline = self
        return self

    def __exit__(self, exception_type, exception_value, traceback):
        Pipeline._current_pipeline = None

    def set_seed(self, seed=0):
        return b.setSeed(seed)

    def create_int_param(self, value=1):
        return b.createIntParameter(value)

    def create_float_param(self, value=1):
        return b.createFloatParameter(value)

    def update_int_param(self, value=1, param=1):
        b.updateIntParameter(value, param)

    def update_float_param(self, value=1, param=1):
        b.updateFloatParameter(value, param)

    def get_int_value(self, param):
        return b.getIntValue(param)

    def get_float_value(self, param):
        return b.getFloatValue(param)

    def get_handle(self):
        return self._handle

    def set_outputs(self, *output_list):
        self._outputs = list(output_list)
        b.setOutputs(self._handle, len(output_list), output_list)

    def build(self):
        status = b.rocalVerify(self._handle)
        if status != types.OK:
            raise RuntimeError("Verify graph failed: " + b.getErrorMessage(self._handle))
        return self

    def rocal_run(self):
        """Enqueues one batch on the pipeline's stream and returns; get_output_tensors() (or wait_on_stream) is where the
        consumer waits for it, as in the reference (pipeline.py: rocal_run, then get_output_tensors in the iterators)."""
        status = b.rocalRun(self._handle)
        if status != types.OK:
            raise RuntimeError("rocalRun failed: " + b.getErrorMessage(self._handle))
        return status

    def get_output_tensors(self):
        """Waits for the batch of the last rocal_run and returns the output tensors (rocAL_pybind/amd/rocal/pipeline.py:
        get_output_tensors). A tensor bound with bind_output is complete in the caller's memory from here on."""
        return b.getOutputTensors(self._handle)

    def wait_on_stream(self, stream=None):
        """Makes a HIP stream (a torch.cuda.Stream, default: torch's current stream) wait for the batch of the last rocal_run
        instead of the host: work queued on it afterwards sees the outputs."""
        import torch
        s = stream if stream is not None else torch.cuda.current_stream()
        if b.outputsWaitOnStream(self._handle, s.cuda_stream) != types.OK:
            raise RuntimeError("wait_on_stream failed: " + b.getErrorMessage(self._handle))

    def set_bilinear_edge_rule(self, device_rule):
        """True: bilinear resizes clamp the right / lower neighbour at the last-but-one pixel of the window, as the reference's
        device kernel does; False (default): at the last pixel. Before the first resize node is added."""
        if b.setBilinearEdgeRule(self._handle, device_rule) != types.OK:
            raise RuntimeError("set_bilinear_edge_rule failed: " + b.getErrorMessage(self._handle))

    def copyToExternalTensor(self, array, multiplier, offset, reverse_channels, tensor_format, tensor_dtype, max_roi_height=0, max_roi_width=0):
        import ctypes
        b.rocalToTensor(self._handle, ctypes.c_void_p(array.data_ptr()), tensor_format, tensor_dtype, multiplier[0], multiplier[1], multiplier[2],
                        offset[0], offset[1], offset[2], reverse_channels, self._output_memory_type, max_roi_height, max_roi_width)

    def timing_info(self):
        return b.getTimingInfo(self._handle)

    # ---- decoded batches in device memory (where the reference has readers and decoders)
    def device_source(self, max_width, max_height, is_output=False):
        return b.deviceSource(self._handle, max_width, max_height, is_output)

    def feed(self, source, tensor, widths, heights):
        """tensor: a torch CUDA uint8 tensor [N, max_height, max_width, 3]; widths / heights: the valid size of each image
        (sequences of integers, or contiguous uint32 numpy arrays, which are passed on as they are)."""
        assert tensor.is_cuda and tensor.is_contiguous()
        self._fed = tensor  # kept alive until the next batch
        status = b.deviceSourceFeed(self._handle, source, tensor.data_ptr(), widths, heights)
        if status != types.OK:
            raise RuntimeError("feed failed: " + b.getErrorMessage(self._handle))

    # ---- decoded images from a loader, batch by batch through a ring of packed pinned / device buffers
    def packed_source(self, max_width, max_height, queue_depth=2, slot_bytes=0, is_output=False):
        """A source fed image by image (place_image) and batch by batch (push): stands where the reference's loader copies every
        decoded image into a padded batch. One asynchronous copy of the bytes written per batch; run() consumes the oldest batch."""
        src = b.packedSource(self._handle, max_width, max_height, is_output, queue_depth, slot_bytes)
        if not src:
            raise RuntimeError("packed_source failed: " + b.getErrorMessage(self._handle))
        return src

    def place_image(self, source, index, image):
        """image: numpy uint8 [h, w, 3], written into the pinned slot of the batch being assembled (rows at dword pitch)."""
        import ctypes as C
        import numpy as np
        image = np.ascontiguousarray(image, dtype=np.uint8)
        h, w, c = image.shape
        assert c == 3
        ptr, stride = b.packedSourcePlaceImage(self._handle, source, index, w, h)
        if not ptr:
            raise RuntimeError("place_image failed: " + b.getErrorMessage(self._handle))
        dst = np.ctypeslib.as_array((C.c_ubyte * (stride * h)).from_address(ptr)).reshape(h, stride)
        dst[:, :3 * w] = image.reshape(h, 3 * w)

    def push(self, source):
        if b.packedSourcePush(self._handle, source) != types.OK:
            raise RuntimeError("push failed: " + b.getErrorMessage(self._handle))

    def wait_for_batch(self, source):
        """Blocks until the loader has pushed a batch (rocal_run on an empty ring raises instead of blocking)."""
        if b.packedSourceWait(self._handle, source) != types.OK:
            raise RuntimeError("wait_for_batch failed: " + b.getErrorMessage(self._handle))

    def stop_source(self, source):
        """Wakes a loader thread blocked in place_image and a consumer blocked in wait_for_batch; they, and every later caller,
        get an exception. release() does this for every packed source before it frees anything."""
        return b.packedSourceStop(self._handle, source)

    def queued_batches(self, source):
        return b.packedSourceLevel(self._handle, source)

    def bind_output(self, output, tensor):
        """The node that produces `output` writes straight into `tensor` (a torch CUDA tensor the caller owns): no copy afterwards."""
        assert tensor.is_cuda and tensor.is_contiguous() and tensor.numel() * tensor.element_size() >= b.tensorDataSize(output)
        self._bound = getattr(self, "_bound", {})
        self._bound[output] = tensor
        if b.tensorSetBuffer(self._handle, output, tensor.data_ptr()) != types.OK:
            raise RuntimeError("bind_output failed: " + b.getErrorMessage(self._handle))

    def output_dlpack(self, output):
        """A DLPack capsule of an output tensor: `torch.from_dlpack(pipe.output_dlpack(out))` aliases the buffer the last node
        wrote (no copy); valid until the next run writes it again. With bind_output the direction is the other way round (the
        node writes into the consumer's tensor)."""
        from . import dlpack
        dims, _, dtype = b.tensorInfo(output)
        ptr = b.tensorBuffer(output)
        if not ptr:
            raise RuntimeError("the tensor has no buffer yet (build the pipeline first)")
        return dlpack.to_dlpack(ptr, dims, dtype, self._device_id, keep_alive=self)

    def output_roi(self, output):
        return b.tensorRoi(output, self._batch_size)

    def release(self):
        if self._handle:
            b.rocalRelease(self._handle)
            self._handle = None
