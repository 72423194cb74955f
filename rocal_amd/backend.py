"""The object the Python API calls `b`: the method names and positional argument orders of the reference's pybind module
(rocAL_pybind/rocal_pybind.cpp), bound with ctypes to the rocal* entry points of librocal_mi355x_host.so. Parameters and
tensors are opaque handles (integers)."""
import ctypes as C
import os

from . import _lib

_HOST = None
_vp, _b, _u, _i, _f = C.c_void_p, C.c_bool, C.c_uint, C.c_int, C.c_float

# name -> (restype, argtypes) of the entry points called directly
_SIGS = {
    "rocalCreate": (_vp, [C.c_size_t, _i, _i, C.c_size_t, C.c_size_t, _i]),
    "rocalVerify": (_i, [_vp]), "rocalRun": (_i, [_vp]), "rocalRelease": (_i, [_vp]), "rocalGetErrorMessage": (C.c_char_p, [_vp]),
    "rocalSetSeed": (None, [_u]), "rocalGetSeed": (_u, []),
    "rocalCreateIntParameter": (_vp, [_i]), "rocalCreateFloatParameter": (_vp, [_f]),
    "rocalCreateIntUniformRand": (_vp, [_i, _i]), "rocalCreateFloatUniformRand": (_vp, [_f, _f]),
    "rocalCreateIntRand": (_vp, [_vp, _vp, _u]), "rocalCreateFloatRand": (_vp, [_vp, _vp, _u]),
    "rocalUpdateIntParameter": (_i, [_i, _vp]), "rocalUpdateFloatParameter": (_i, [_f, _vp]),
    "rocalGetIntValue": (_i, [_vp]), "rocalGetFloatValue": (_f, [_vp]),
    "rocalDeviceSource": (_vp, [_vp, _u, _u, _b]), "rocalDeviceSourceFeed": (_i, [_vp, _vp, _vp, _vp, _vp]),
    "rocalPackedSource": (_vp, [_vp, _u, _u, _b, _u, C.c_size_t]),
    "rocalPackedSourcePlaceImage": (_vp, [_vp, _vp, _u, _u, _u, C.POINTER(_u)]),
    "rocalPackedSourcePush": (_i, [_vp, _vp]), "rocalPackedSourceWait": (_i, [_vp, _vp]), "rocalPackedSourceLevel": (C.c_size_t, [_vp, _vp]),
    "rocalPackedSourceStop": (_i, [_vp, _vp]), "rocalSetBilinearEdgeRule": (_i, [_vp, _i]), "rocalOutputsWaitOnStream": (_i, [_vp, _vp]),
    "rocalCopyToOutput": (_i, [_vp, _vp, C.c_size_t]), "rocalpy_output_tensors": (_i, [_vp, _vp, _u]),
    "rocalTensorBuffer": (_vp, [_vp]), "rocalTensorRoi": (C.POINTER(_u), [_vp]), "rocalTensorDataSize": (C.c_size_t, [_vp]),
    "rocalTensorSetBuffer": (_i, [_vp, _vp, _vp]),
    "rocalTensorInfo": (_i, [_vp, C.POINTER(C.c_size_t), C.POINTER(_i), C.POINTER(_i)]),
    "rocalToTensor": (_i, [_vp, _vp, _i, _i, _f, _f, _f, _f, _f, _f, _b, _i, _i, _i]),
    "rocalCropResize": (_vp, [_vp, _vp, _u, _u, _b, _vp, _vp, _vp, _vp, _i, _i]),
    "rocalROIResize": (_vp, [_vp, _vp, _u, _u, _b, _u, _u, _f, _f, _i, _i, _i]),
    "rocalRotate": (_vp, [_vp, _vp, _b, _vp, _u, _u, _i, _i, _i]),
    "rocalBrightness": (_vp, [_vp, _vp, _b, _vp, _vp, _i, _i]), "rocalBrightnessFixed": (_vp, [_vp, _vp, _f, _f, _b, _i, _i]),
    "rocalContrast": (_vp, [_vp, _vp, _b, _vp, _vp, _i, _i]),
    "rocalFlip": (_vp, [_vp, _vp, _b, _vp, _vp, _i, _i]),
    "rocalWarpAffineFixed": (_vp, [_vp, _vp, _f, _f, _f, _f, _f, _f, _b, _u, _u, _i, _i, _i]),
    "rocalHue": (_vp, [_vp, _vp, _b, _vp, _i, _i]), "rocalSaturation": (_vp, [_vp, _vp, _b, _vp, _i, _i]),
    "rocalColorTwist": (_vp, [_vp, _vp, _b, _vp, _vp, _vp, _vp, _i, _i]),
    "rocalGamma": (_vp, [_vp, _vp, _b, _vp, _i, _i]), "rocalExposure": (_vp, [_vp, _vp, _b, _vp, _i, _i]),
    "rocalColorTemp": (_vp, [_vp, _vp, _b, _vp, _i, _i]), "rocalBlend": (_vp, [_vp, _vp, _vp, _b, _vp, _i, _i]),
    "rocalCrop": (_vp, [_vp, _vp, _b, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i]),
    "rocalCropFixed": (_vp, [_vp, _vp, _u, _u, _u, _b, _f, _f, _f, _i, _i]),
    "rocalCropCenterFixed": (_vp, [_vp, _vp, _u, _u, _u, _b, _i, _i]),
    "rocalResizeCropMirrorFixed": (_vp, [_vp, _vp, _u, _u, _b, _u, _u, _vp, _i, _i]),
    "rocalRandomCrop": (_vp, [_vp, _vp, _b, _vp, _vp, _vp, _vp, _i, _i, _i]),
    "rocalpy_resize": (_vp, [_vp, _vp, _u, _u, _b, _i, _vp, _u, _u, _u, _i, _i, _i]),
    "rocalpy_resize_mirror_normalize": (_vp, [_vp, _vp, _u, _u, _vp, _u, _vp, _u, _b, _i, _vp, _u, _u, _u, _i, _vp, _i, _i]),
    "rocalpy_crop_mirror_normalize": (_vp, [_vp, _vp, _u, _u, _f, _f, _vp, _u, _vp, _u, _b, _vp, _i, _i]),
    "rocalpy_normalize": (_vp, [_vp, _vp, _vp, _u, _vp, _u, _vp, _u, _b, _f, _f, _i]),
    "rocalpy_transpose": (_vp, [_vp, _vp, _vp, _u, _b, _i]),
    "rocalpy_set_outputs": (_i, [_vp, _u, _vp]), "rocalpy_timing": (None, [_vp, _vp]),
}


def host():
    """Loads librocal_mi355x_host.so (raises if it has not been built)."""
    global _HOST
    if _HOST is None:
        _lib.lib()  # the C-ABI library first: one HIP runtime instance for both
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "librocal_mi355x_host.so")
        if not os.path.exists(path):
            raise _lib.RmxError(-1, "host library not built: %s is missing (run `make -C rocal_amd/host`)" % path)
        h = C.CDLL(path)
        for name, (res, args) in _SIGS.items():
            fn = getattr(h, name)
            fn.restype, fn.argtypes = res, args
        _HOST = h
    return _HOST


def _farr(v):
    a = (C.c_float * len(v))(*[float(x) for x in v])
    return a, len(v)


def _uarr(v):
    v = [v] if isinstance(v, int) else list(v)
    a = (C.c_uint * max(len(v), 1))(*[int(x) for x in v])
    return (a if v else None), len(v)


class Backend:
    """Method names of the reference's pybind module; as there, every augmentation method takes its arguments in the order of
    the C entry point it is bound to (rocal_pybind.cpp:1072-1135 binds the functions themselves)."""

    # context
    def rocalCreate(self, batch_size, affinity, gpu_id, cpu_threads, prefetch_queue_depth, output_dtype):
        return host().rocalCreate(batch_size, affinity, gpu_id, max(cpu_threads, 1), prefetch_queue_depth, output_dtype)

    def getStatus(self, handle):
        return 0 if handle else 2

    def rocalVerify(self, handle):
        return host().rocalVerify(handle)

    def rocalRun(self, handle):
        return host().rocalRun(handle)

    def rocalRelease(self, handle):
        return host().rocalRelease(handle)

    def setBilinearEdgeRule(self, handle, device_rule):
        return host().rocalSetBilinearEdgeRule(handle, 1 if device_rule else 0)

    def getOutputTensors(self, handle):
        """rocalGetOutputTensors: waits for the batch of the last run and returns the handles of the output tensors."""
        arr = (C.c_void_p * 64)()
        n = host().rocalpy_output_tensors(handle, arr, 64)
        if n < 0:
            raise RuntimeError("rocalGetOutputTensors failed: " + self.getErrorMessage(handle))
        return [arr[i] for i in range(n)]

    def outputsWaitOnStream(self, handle, stream):
        return host().rocalOutputsWaitOnStream(handle, stream)

    def copyToOutput(self, handle, ptr, size):
        return host().rocalCopyToOutput(handle, ptr, size)

    def getErrorMessage(self, handle):
        return host().rocalGetErrorMessage(handle).decode()

    def setOutputs(self, handle, n, tensors):
        arr = (C.c_void_p * n)(*tensors)
        if host().rocalpy_set_outputs(handle, n, arr) != 0:
            raise RuntimeError("rocalSetOutputs failed")

    def getTimingInfo(self, handle):
        t = (C.c_ulonglong * 5)()
        host().rocalpy_timing(handle, t)
        return {"load_time": t[0], "decode_time": t[1], "process_time": t[2], "transfer_time": t[3], "parameter_update_time": t[4]}

    def rocalToTensor(self, handle, ptr, layout, dtype, m0, m1, m2, o0, o1, o2, reverse_channels, mem_type, max_roi_height=0, max_roi_width=0):
        return host().rocalToTensor(handle, ptr, layout, dtype, m0, m1, m2, o0, o1, o2, reverse_channels, mem_type, max_roi_height, max_roi_width)

    # parameters
    def setSeed(self, seed):
        host().rocalSetSeed(seed)

    def getSeed(self):
        return host().rocalGetSeed()

    def createIntParameter(self, v):
        return host().rocalCreateIntParameter(v)

    def createFloatParameter(self, v):
        return host().rocalCreateFloatParameter(v)

    def createIntUniformRand(self, start, end):
        return host().rocalCreateIntUniformRand(start, end)

    def createFloatUniformRand(self, start, end):
        return host().rocalCreateFloatUniformRand(start, end)

    def createIntRand(self, values, frequencies, size):
        v = (C.c_int * size)(*values)
        f = (C.c_double * size)(*frequencies)
        return host().rocalCreateIntRand(v, f, size)

    def updateIntParameter(self, v, p):
        return host().rocalUpdateIntParameter(v, p)

    def updateFloatParameter(self, v, p):
        return host().rocalUpdateFloatParameter(v, p)

    def getIntValue(self, p):
        return host().rocalGetIntValue(p)

    def getFloatValue(self, p):
        return host().rocalGetFloatValue(p)

    # decoded batches in device memory (stands where readers + decoders stand)
    def deviceSource(self, handle, max_width, max_height, is_output):
        return host().rocalDeviceSource(handle, max_width, max_height, is_output)

    def deviceSourceFeed(self, handle, source, device_ptr, widths, heights):
        # contiguous uint32 numpy arrays are handed over as they are (no per-element conversion on the per-batch path)
        def as_uints(v):
            if hasattr(v, "ctypes") and getattr(v, "dtype", None) == "uint32" and v.flags["C_CONTIGUOUS"] and v.ndim == 1:
                return v.ctypes.data_as(C.POINTER(C.c_uint)), v
            arr = (C.c_uint * len(v))(*[int(x) for x in v])
            return arr, arr
        w, keep_w = as_uints(widths)
        h, keep_h = as_uints(heights)
        if len(widths) != len(heights):
            raise ValueError("widths and heights differ in length")
        return host().rocalDeviceSourceFeed(handle, source, device_ptr, w, h)

    def packedSource(self, handle, max_width, max_height, is_output, queue_depth, slot_bytes):
        return host().rocalPackedSource(handle, max_width, max_height, is_output, queue_depth, slot_bytes)

    def packedSourcePlaceImage(self, handle, source, index, width, height):
        """Returns (address of the image's first row in pinned host memory, row stride in bytes); address 0 on error."""
        stride = _u(0)
        p = host().rocalPackedSourcePlaceImage(handle, source, index, width, height, C.byref(stride))
        return (p or 0), int(stride.value)

    def packedSourcePush(self, handle, source):
        return host().rocalPackedSourcePush(handle, source)

    def packedSourceWait(self, handle, source):
        return host().rocalPackedSourceWait(handle, source)

    def packedSourceStop(self, handle, source):
        return host().rocalPackedSourceStop(handle, source)

    def packedSourceLevel(self, handle, source):
        return int(host().rocalPackedSourceLevel(handle, source))

    def tensorBuffer(self, t):
        return host().rocalTensorBuffer(t)

    def tensorSetBuffer(self, handle, t, ptr):
        return host().rocalTensorSetBuffer(handle, t, ptr)

    def tensorDataSize(self, t):
        return host().rocalTensorDataSize(t)

    def tensorInfo(self, t):
        """(dims in the order of the layout, layout, data type)"""
        dims = (C.c_size_t * 4)()
        layout, dtype = _i(0), _i(0)
        if host().rocalTensorInfo(t, dims, C.byref(layout), C.byref(dtype)) != 0:
            raise ValueError("not a tensor")
        return [int(d) for d in dims], int(layout.value), int(dtype.value)

    def tensorRoi(self, t, n):
        p = host().rocalTensorRoi(t)
        return [[p[4 * i + k] for k in range(4)] for i in range(n)]

    # augmentations: (handle, input, ...) in the order of the reference's pybind lambdas = the C API's
    def resize(self, handle, inp, dest_width, dest_height, is_output, scaling_mode, max_size, resize_shorter, resize_longer, interpolation, layout, dtype):
        ms, n = _uarr(max_size)
        return host().rocalpy_resize(handle, inp, dest_width, dest_height, is_output, scaling_mode, ms, n, resize_shorter, resize_longer, interpolation, layout, dtype)

    def resizeMirrorNormalize(self, handle, inp, dest_width, dest_height, mean, std_dev, is_output, scaling_mode, max_size, resize_shorter,
                              resize_longer, interpolation, mirror, layout, dtype):
        (m, nm), (s, ns), (ms, n) = _farr(mean), _farr(std_dev), _uarr(max_size)
        return host().rocalpy_resize_mirror_normalize(handle, inp, dest_width, dest_height, m, nm, s, ns, is_output, scaling_mode, ms, n,
                                                      resize_shorter, resize_longer, interpolation, mirror, layout, dtype)

    def cropMirrorNormalize(self, handle, inp, crop_height, crop_width, start_x, start_y, mean, std_dev, is_output, mirror, layout, dtype):
        (m, nm), (s, ns) = _farr(mean), _farr(std_dev)
        return host().rocalpy_crop_mirror_normalize(handle, inp, crop_height, crop_width, start_x, start_y, m, nm, s, ns, is_output, mirror, layout, dtype)

    def cropResize(self, handle, inp, dest_width, dest_height, is_output, area, aspect_ratio, x_drift, y_drift, layout, dtype):
        return host().rocalCropResize(handle, inp, dest_width, dest_height, is_output, area, aspect_ratio, x_drift, y_drift, layout, dtype)

    def roiResize(self, handle, inp, dest_width, dest_height, is_output, roi_h, roi_w, roi_pos_x, roi_pos_y, interpolation, layout, dtype):
        return host().rocalROIResize(handle, inp, dest_width, dest_height, is_output, roi_h or 0, roi_w or 0, roi_pos_x or 0.0, roi_pos_y or 0.0,
                                     interpolation, layout, dtype)

    def resizeCropMirrorFixed(self, handle, inp, dest_width, dest_height, is_output, crop_h, crop_w, mirror, layout, dtype):
        return host().rocalResizeCropMirrorFixed(handle, inp, dest_width, dest_height, is_output, crop_h, crop_w, mirror, layout, dtype)

    def randomCrop(self, handle, inp, is_output, area, aspect_ratio, pos_x, pos_y, num_attempts, layout, dtype):
        return host().rocalRandomCrop(handle, inp, is_output, area, aspect_ratio, pos_x, pos_y, num_attempts, layout, dtype)

    def rotate(self, handle, inp, is_output, angle, dest_width, dest_height, interpolation, layout, dtype):
        return host().rocalRotate(handle, inp, is_output, angle, dest_width, dest_height, interpolation, layout, dtype)

    def warpAffineFixed(self, handle, inp, x0, x1, y0, y1, o0, o1, is_output, dest_height, dest_width, interpolation, layout, dtype):
        return host().rocalWarpAffineFixed(handle, inp, x0, x1, y0, y1, o0, o1, is_output, dest_height, dest_width, interpolation, layout, dtype)

    def brightness(self, handle, inp, is_output, alpha, beta, layout, dtype):
        return host().rocalBrightness(handle, inp, is_output, alpha, beta, layout, dtype)

    def brightnessFixed(self, handle, inp, alpha, beta, is_output, layout, dtype):
        return host().rocalBrightnessFixed(handle, inp, alpha, beta, is_output, layout, dtype)

    def contrast(self, handle, inp, is_output, factor, center, layout, dtype):
        return host().rocalContrast(handle, inp, is_output, factor, center, layout, dtype)

    def flip(self, handle, inp, is_output, horizontal, vertical, layout, dtype):
        return host().rocalFlip(handle, inp, is_output, horizontal, vertical, layout, dtype)

    def hue(self, handle, inp, is_output, hue, layout, dtype):
        return host().rocalHue(handle, inp, is_output, hue, layout, dtype)

    def saturation(self, handle, inp, is_output, sat, layout, dtype):
        return host().rocalSaturation(handle, inp, is_output, sat, layout, dtype)

    def colorTwist(self, handle, inp, is_output, alpha, beta, hue, sat, layout, dtype):
        return host().rocalColorTwist(handle, inp, is_output, alpha, beta, hue, sat, layout, dtype)

    def gammaCorrection(self, handle, inp, is_output, gamma, layout, dtype):
        return host().rocalGamma(handle, inp, is_output, gamma, layout, dtype)

    def exposure(self, handle, inp, is_output, factor, layout, dtype):
        return host().rocalExposure(handle, inp, is_output, factor, layout, dtype)

    def colorTemp(self, handle, inp, is_output, adjustment, layout, dtype):
        return host().rocalColorTemp(handle, inp, is_output, adjustment, layout, dtype)

    def blend(self, handle, inp1, inp2, is_output, ratio, layout, dtype):
        return host().rocalBlend(handle, inp1, inp2, is_output, ratio, layout, dtype)

    def normalize(self, handle, inp, axes, mean, std_dev, is_output, scale, shift, dtype):
        (ax, na), (m, nm), (s, ns) = _uarr(axes), _farr(mean), _farr(std_dev)
        return host().rocalpy_normalize(handle, inp, ax, na, m if nm else None, nm, s if ns else None, ns, is_output, scale, shift, dtype)

    def transpose(self, handle, inp, perm, is_output, layout):
        p, n = _uarr(perm)
        return host().rocalpy_transpose(handle, inp, p, n, is_output, layout)

    def crop(self, handle, inp, is_output, crop_width, crop_height, crop_depth, pos_x, pos_y, pos_z, layout, dtype):
        return host().rocalCrop(handle, inp, is_output, crop_width, crop_height, crop_depth, pos_x, pos_y, pos_z, layout, dtype)

    def cropFixed(self, handle, inp, crop_width, crop_height, crop_depth, is_output, pos_x, pos_y, pos_z, layout, dtype):
        return host().rocalCropFixed(handle, inp, crop_width, crop_height, crop_depth, is_output, pos_x, pos_y, pos_z, layout, dtype)

    def centerCropFixed(self, handle, inp, crop_width, crop_height, crop_depth, is_output, layout, dtype):
        return host().rocalCropCenterFixed(handle, inp, crop_width, crop_height, crop_depth, is_output, layout, dtype)
