"""Thin Python doorway onto the C ABI (include/rocal_mi355x.h): contexts and per-node ops.

torch is used only for device memory and streams; every pixel is produced by the HIP kernels
in librocal_mi355x.so. Parameter arrays are numpy (host) arrays, as rocAL's vx_arrays are.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import TensorDesc, check

NHWC, NCHW = 0, 1
FP32, FP16, UINT8 = 0, 1, 2
ROI_LTRB, ROI_XYWH = 0, 1
NEAREST, LINEAR, TRIANGULAR = 0, 1, 5
F_QUANTIZE_U8 = 1
F_COLOR_LINEAR, F_COLOR_TWIST = 2, 4
F_EDGE_REF = 8  # bilinear neighbours clamp to the window's last-but-one column / row, as the reference's device code does


def _torch():
    import torch
    return torch


def torch_dtype(dtype):
    t = _torch()
    return {FP32: t.float32, FP16: t.float16, UINT8: t.uint8}[dtype]


def _arr(a, dt):
    if a is None:
        return None, None
    a = np.ascontiguousarray(a, dtype=dt)
    return a, a.ctypes.data_as(C.c_void_p)


class Context:
    """One device + one stream (rmx_ctx). stream="torch" borrows torch's current stream,
    stream="own" lets the context create its own, an integer is a hipStream_t to borrow."""

    def __init__(self, device=0, stream="torch"):
        self._h = C.c_void_p()
        sp, own = None, 0
        if stream == "torch":
            t = _torch()
            sp = C.c_void_p(t.cuda.current_stream(device).cuda_stream)
        elif stream == "own":
            own = 1
        elif stream is not None:
            sp = C.c_void_p(int(stream))
        check(_lib.lib().rmx_ctx_create(int(device), sp, own, C.byref(self._h)))
        self.device = device

    def sync(self):
        check(_lib.lib().rmx_ctx_sync(self._h))

    @property
    def stream(self):
        return _lib.lib().rmx_ctx_stream(self._h)

    def copy_bytes(self, src, dst, nbytes):
        check(_lib.lib().rmx_copy_bytes(self._h, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), nbytes))

    def stream_probe(self, mode, src, dst, nbytes, groups_per_cu=0):
        """One streaming pass: mode 0 copies src to dst, 1 only reads src, 2 only writes dst."""
        check(_lib.lib().rmx_stream_probe(self._h, mode, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), nbytes, groups_per_cu))

    def close(self):
        if self._h:
            _lib.lib().rmx_ctx_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def desc(n, h, w, layout, dtype, c=3):
    return TensorDesc(n, h, w, c, layout, dtype)


NOALLOC_MAX_SAMPLES = 512  # RMX_NOALLOC_MAX_SAMPLES


def resize_cmn_noalloc(ctx, src_desc, dst_desc, src, dst, src_roi, dst_w, dst_h, scale, bias, mirror=None, crop_roi=None,
                       interpolation=LINEAR, flags=0, roi_type=ROI_XYWH):
    """rmx_resize_cmn_noalloc: the fused chain resize -> CropMirrorNormalize in one call that allocates nothing (the parameter
    table lives in a static device array). src / dst: torch CUDA tensors, the arrays are host arrays."""
    assert src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()
    assert src.numel() * src.element_size() >= src_desc.n * src_desc.h * src_desc.w * src_desc.c
    esz = {FP32: 4, FP16: 2, UINT8: 1}[dst_desc.dtype]
    assert dst.numel() * dst.element_size() >= dst_desc.n * dst_desc.h * dst_desc.w * dst_desc.c * esz
    keep = [_arr(a, dt) for a, dt in ((src_roi, _U), (dst_w, _U), (dst_h, _U), (crop_roi, _U), (scale, _F), (bias, _F), (mirror, _U))]
    check(_lib.lib().rmx_resize_cmn_noalloc(ctx._h, C.byref(src_desc), C.byref(dst_desc), int(interpolation), int(roi_type), C.c_uint32(flags),
                                            C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), *[p for _, p in keep]))


class Op:
    """One node (rmx_op). Subclasses bind create/update of a specific reference node."""

    _create = None

    def __init__(self, ctx, src_desc, dst_desc, *extra, roi_type=ROI_XYWH):
        self.ctx = ctx
        self.src_desc, self.dst_desc = src_desc, dst_desc
        self._h = C.c_void_p()
        fn = getattr(_lib.lib(), self._create)
        check(fn(ctx._h, C.byref(src_desc), C.byref(dst_desc), *extra[:self._n_pre], int(roi_type),
                 *extra[self._n_pre:], C.byref(self._h)))

    _n_pre = 0

    def _update(self, name, *arrays_and_types):
        keep, ptrs = [], []
        for a, dt in arrays_and_types:
            arr, p = _arr(a, dt)
            keep.append(arr)
            ptrs.append(p)
        fn = getattr(_lib.lib(), name)
        self._last_update = (fn, keep, ptrs)
        check(fn(self._h, *ptrs))

    def prepared_update(self):
        """A zero-argument callable that repeats the last update with the same (already converted) host arrays:
        the C-ABI call alone, without numpy conversions - what a C++ caller pays per batch."""
        fn, keep, ptrs = self._last_update
        h = self._h

        def call(_keep=keep):
            check(fn(h, *ptrs))
        return call

    def prepared_launch(self, src, dst):
        """A zero-argument callable that launches on these two batch buffers (checked once, here)."""
        assert src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()
        fn, h, ps, pd = _lib.lib().rmx_op_launch, self._h, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr())

        def call(_keep=(src, dst)):
            check(fn(h, ps, pd))
        return call

    def launch(self, src, dst):
        """src/dst: torch CUDA tensors (the batch buffers). Asynchronous on the context's stream."""
        assert src.is_cuda and dst.is_cuda and src.is_contiguous() and dst.is_contiguous()
        sd, dd = self.src_desc, self.dst_desc
        need = getattr(self, "_ragged_bytes", None) or sd.n * sd.h * sd.w * sd.c
        assert src.numel() * src.element_size() >= need, "source buffer smaller than its descriptor"
        esz = {FP32: 4, FP16: 2, UINT8: 1}[dd.dtype]
        assert dst.numel() * dst.element_size() >= dd.n * dd.h * dd.w * dd.c * esz, "destination buffer smaller than its descriptor"
        check(_lib.lib().rmx_op_launch(self._h, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr())))

    def alloc_output(self, fill=0):
        t = _torch()
        d = self.dst_desc
        shape = (d.n, d.c, d.h, d.w) if d.layout == NCHW else (d.n, d.h, d.w, d.c)
        return t.full(shape, fill, dtype=torch_dtype(d.dtype), device="cuda:%d" % self.ctx.device)

    def set_ragged_source(self, offsets, widths, heights, buffer_bytes, row_strides=None):
        """The batch's images lie packed at byte `offsets` of one buffer, rows `row_strides` bytes apart (default: width*3, no
        padding at all); offsets None: padded tensor again."""
        if offsets is None:
            check(_lib.lib().rmx_op_set_ragged_source(self._h, None, None, None, 0))
            self._ragged_bytes = None
            return
        self._ragged_bytes = int(buffer_bytes)
        o = np.ascontiguousarray(offsets, np.uint64)
        w = np.ascontiguousarray(widths, np.uint32)
        h = np.ascontiguousarray(heights, np.uint32)
        if row_strides is None:
            check(_lib.lib().rmx_op_set_ragged_source(self._h, o.ctypes.data_as(C.c_void_p), w.ctypes.data_as(C.c_void_p), h.ctypes.data_as(C.c_void_p),
                                                      int(buffer_bytes)))
        else:
            st = np.ascontiguousarray(row_strides, np.uint32)
            check(_lib.lib().rmx_op_set_ragged_source_strided(self._h, o.ctypes.data_as(C.c_void_p), w.ctypes.data_as(C.c_void_p),
                                                              h.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p), int(buffer_bytes)))

    @property
    def algorithmic_bytes(self):
        return int(_lib.lib().rmx_op_algorithmic_bytes(self._h))

    @property
    def kernel_name(self):
        return _lib.lib().rmx_op_kernel_name(self._h).decode()

    @property
    def plan(self):
        return _lib.lib().rmx_op_plan(self._h).decode()

    def close(self):
        if self._h:
            _lib.lib().rmx_op_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


_U, _F = np.uint32, np.float32


class CropMirrorNormalize(Op):
    _create = "rmx_create_crop_mirror_normalize"

    def update(self, crop_roi, scale, bias, mirror=None):
        self._update("rmx_update_crop_mirror_normalize", (crop_roi, _U), (scale, _F), (bias, _F), (mirror, _U))


class Crop(Op):
    _create = "rmx_create_crop"

    def update(self, crop_roi):
        self._update("rmx_update_crop", (crop_roi, _U))


class Flip(Op):
    _create = "rmx_create_flip"

    def update(self, src_roi, horizontal, vertical):
        self._update("rmx_update_flip", (src_roi, _U), (horizontal, _U), (vertical, _U))


class ToTensor(Op):
    """MasterGraph::to_tensor / Hip_CopyInt8ToNCHW: whole image, per-channel multiplier/offset, optional RGB<->BGR."""

    def __init__(self, ctx, src_desc, dst_desc):
        self.ctx = ctx
        self.src_desc, self.dst_desc = src_desc, dst_desc
        self._h = C.c_void_p()
        check(_lib.lib().rmx_create_to_tensor(ctx._h, C.byref(src_desc), C.byref(dst_desc), C.byref(self._h)))

    def update(self, multiplier, offset, reverse_channels=False):
        m, pm = _arr(multiplier, _F)
        o, po = _arr(offset, _F)
        assert m.size == 3 and o.size == 3
        check(_lib.lib().rmx_update_to_tensor(self._h, pm, po, int(bool(reverse_channels))))


class Resize(Op):
    _create = "rmx_create_resize"
    _n_pre = 1

    def __init__(self, ctx, src_desc, dst_desc, interpolation=LINEAR, flags=0, roi_type=ROI_XYWH):
        super().__init__(ctx, src_desc, dst_desc, int(interpolation), C.c_uint32(flags), roi_type=roi_type)

    def update(self, src_roi, dst_w, dst_h, mirror=None, mean=None, stddev=None):
        self._update("rmx_update_resize", (src_roi, _U), (dst_w, _U), (dst_h, _U), (mirror, _U), (mean, _F), (stddev, _F))

    def update_cmn(self, src_roi, dst_w, dst_h, scale, bias, mirror=None, crop_roi=None):
        self._update("rmx_update_resize_cmn", (src_roi, _U), (dst_w, _U), (dst_h, _U), (crop_roi, _U), (scale, _F),
                     (bias, _F), (mirror, _U))


    def update_color_cmn(self, src_roi, dst_w, dst_h, scale, bias, colour, mirror=None, crop_roi=None):
        """colour: up to four [N] arrays (None = neutral) of the chain's colour node, see RMX_F_COLOR_LINEAR / _TWIST."""
        c = list(colour) + [None] * (4 - len(colour))
        self._update("rmx_update_resize_color_cmn", (src_roi, _U), (dst_w, _U), (dst_h, _U), (crop_roi, _U), (scale, _F), (bias, _F),
                     (mirror, _U), (c[0], _F), (c[1], _F), (c[2], _F), (c[3], _F))


class ColorTwist(Op):
    _create = "rmx_create_color_twist"

    def update(self, src_roi, alpha, beta, hue, sat):
        self._update("rmx_update_color_twist", (src_roi, _U), (alpha, _F), (beta, _F), (hue, _F), (sat, _F))


class Brightness(Op):
    _create = "rmx_create_brightness"

    def update(self, src_roi, alpha, beta):
        self._update("rmx_update_brightness", (src_roi, _U), (alpha, _F), (beta, _F))


class Contrast(Op):
    _create = "rmx_create_contrast"

    def update(self, src_roi, factor, center):
        self._update("rmx_update_contrast", (src_roi, _U), (factor, _F), (center, _F))


class Hue(Op):
    _create = "rmx_create_hue"

    def update(self, src_roi, hue):
        self._update("rmx_update_hue", (src_roi, _U), (hue, _F))


class Saturation(Op):
    _create = "rmx_create_saturation"

    def update(self, src_roi, sat):
        self._update("rmx_update_saturation", (src_roi, _U), (sat, _F))


class Gamma(Op):
    _create = "rmx_create_gamma"

    def update(self, src_roi, gamma):
        self._update("rmx_update_gamma", (src_roi, _U), (gamma, _F))


class Exposure(Op):
    _create = "rmx_create_exposure"

    def update(self, src_roi, factor):
        self._update("rmx_update_exposure", (src_roi, _U), (factor, _F))


class ColorTemperature(Op):
    _create = "rmx_create_color_temperature"

    def update(self, src_roi, adjustment):
        self._update("rmx_update_color_temperature", (src_roi, _U), (adjustment, np.int32))


class Normalize(Op):
    """Per-sample normalisation over height and width (axis_mask 3) or height, width and channels (7); mean / stddev None = computed."""
    _create = "rmx_create_normalize"

    def update(self, src_roi, axis_mask=3, mean=None, stddev=None, scale=1.0, shift=0.0):
        roi, proi = _arr(src_roi, _U)
        m, pm = _arr(mean, _F)
        s, ps = _arr(stddev, _F)
        n_stats = m.size if m is not None else (s.size if s is not None else 0)
        if m is not None and s is not None:
            assert m.size == s.size
        check(_lib.lib().rmx_update_normalize(self._h, proi, int(axis_mask), pm, ps, int(n_stats), float(scale), float(shift)))


class Transpose(Op):
    """perm: the source's (height, width, channels) axes in output order: (0,1,2), (2,0,1), (1,0,2) or (2,1,0)."""

    def __init__(self, ctx, src_desc, dst_desc, perm, roi_type=ROI_XYWH):
        self.ctx = ctx
        self.src_desc, self.dst_desc = src_desc, dst_desc
        self._h = C.c_void_p()
        p = np.ascontiguousarray(perm, np.uint32)
        check(_lib.lib().rmx_create_transpose(ctx._h, C.byref(src_desc), C.byref(dst_desc), p.ctypes.data_as(C.c_void_p), int(roi_type), C.byref(self._h)))

    def update(self, src_roi=None):
        self._update("rmx_update_transpose", (src_roi, _U))


class Blend(Op):
    """Two source batches of one shape; launch(src1, src2, dst)."""
    _create = "rmx_create_blend"

    def update(self, src_roi, ratio):
        self._update("rmx_update_blend", (src_roi, _U), (ratio, _F))

    def launch(self, src1, src2, dst):
        assert src1.is_cuda and src2.is_cuda and dst.is_cuda and src1.is_contiguous() and src2.is_contiguous() and dst.is_contiguous()
        sd, dd = self.src_desc, self.dst_desc
        need = sd.n * sd.h * sd.w * sd.c
        assert src1.numel() * src1.element_size() >= need and src2.numel() * src2.element_size() >= need, "source buffer smaller than its descriptor"
        esz = {FP32: 4, FP16: 2, UINT8: 1}[dd.dtype]
        assert dst.numel() * dst.element_size() >= dd.n * dd.h * dd.w * dd.c * esz, "destination buffer smaller than its descriptor"
        check(_lib.lib().rmx_op_launch2(self._h, C.c_void_p(src1.data_ptr()), C.c_void_p(src2.data_ptr()), C.c_void_p(dst.data_ptr())))


class WarpAffine(Op):
    _create = "rmx_create_warp_affine"
    _n_pre = 1

    def __init__(self, ctx, src_desc, dst_desc, interpolation=LINEAR, roi_type=ROI_XYWH):
        super().__init__(ctx, src_desc, dst_desc, int(interpolation), roi_type=roi_type)

    def update(self, src_roi, affine, dst_w, dst_h):
        self._update("rmx_update_warp_affine", (src_roi, _U), (affine, _F), (dst_w, _U), (dst_h, _U))


class Rotate(Op):
    _create = "rmx_create_rotate"
    _n_pre = 1

    def __init__(self, ctx, src_desc, dst_desc, interpolation=LINEAR, roi_type=ROI_XYWH):
        super().__init__(ctx, src_desc, dst_desc, int(interpolation), roi_type=roi_type)

    def update(self, src_roi, angle, dst_w, dst_h):
        self._update("rmx_update_rotate", (src_roi, _U), (angle, _F), (dst_w, _U), (dst_h, _U))
