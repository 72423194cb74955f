"""ctypes doorway onto the CPU oracle (oracle/rocal_oracle.c). TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's cpu_baseline leg may import this module;
the shipped package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librocal_oracle.so")

NHWC, NCHW = 0, 1
FP32, FP16, UINT8 = 0, 1, 2
NEAREST, LINEAR, TRIANGULAR = 0, 1, 5

F_ROUND_TRUNC = 1 << 0
F_BILINEAR_EDGE_QUIRK = 1 << 1
F_TRI_2D = 1 << 2
F_QUANTIZE_U8 = 1 << 3
F_FP16_TRUNC = 1 << 4
F_HUE_INT_TRUNC = 1 << 5

_NP_DTYPE = {FP32: np.float32, FP16: np.float16, UINT8: np.uint8}


class _Src(C.Structure):
    _fields_ = [("data", C.c_void_p), ("n", C.c_int), ("hmax", C.c_int), ("wmax", C.c_int), ("c", C.c_int)]


class _Dst(C.Structure):
    _fields_ = [("data", C.c_void_p), ("n", C.c_int), ("hmax", C.c_int), ("wmax", C.c_int), ("c", C.c_int),
                ("layout", C.c_int), ("dtype", C.c_int)]


class _MT(C.Structure):
    _fields_ = [("mt", C.c_uint32 * 624), ("idx", C.c_int)]


def build(force=False):
    """Compile the oracle with the recipe beside it (oracle/Makefile)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "librocal_oracle.so"] + (["-B"] if force else []))


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f32_to_f16.restype = C.c_uint16
        _lib.orc_f32_to_f16.argtypes = [C.c_float, C.c_int]
        _lib.orc_f16_to_f32.restype = C.c_float
        _lib.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_uniform_rand_f32.restype = C.c_float
        _lib.orc_uniform_rand_f32.argtypes = [C.c_void_p, C.c_float, C.c_float]
        _lib.orc_uniform_rand_i32.restype = C.c_int
        _lib.orc_uniform_rand_i32.argtypes = [C.c_void_p, C.c_int, C.c_int]
        _lib.orc_mt19937_next.restype = C.c_uint32
        _lib.orc_custom_rand_index.restype = C.c_int
        _lib.orc_fixed_crop.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.c_float,
                                        C.c_float, C.c_uint32, C.c_uint32, C.c_void_p]
        _lib.orc_rotate_matrix.argtypes = [C.c_float, C.c_void_p]
        _lib.orc_gamma_lut.argtypes = [C.c_float, C.c_void_p, C.c_uint]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _u32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.uint32)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def _src(img):
    assert img.dtype == np.uint8 and img.ndim == 4 and img.flags.c_contiguous
    n, h, w, c = img.shape
    return _Src(img.ctypes.data, n, h, w, c)


def _alloc_dst(n, c, h, w, layout, dtype, fill=0):
    shape = (n, c, h, w) if layout == NCHW else (n, h, w, c)
    out = np.full(shape, fill, dtype=_NP_DTYPE[dtype])
    return out, _Dst(out.ctypes.data, n, h, w, c, layout, dtype)


def f32_to_f16(v, trunc=False):
    return int(lib().orc_f32_to_f16(float(v), int(trunc)))


def cmn_scale_bias(mean, std, n):
    mean, std = _f32(mean), _f32(std)
    c = len(mean)
    scale = np.empty(n * c, np.float32)
    bias = np.empty(n * c, np.float32)
    lib().orc_cmn_scale_bias(_p(mean), _p(std), c, n, _p(scale), _p(bias))
    return scale, bias


def crop_mirror_normalize(img, crop_xywh, scale, bias, mirror, out_h, out_w, layout=NCHW, dtype=FP32,
                          vflip=None, flags=0):
    crop_xywh, mirror, vflip = _u32(crop_xywh), _u32(mirror), _u32(vflip)
    scale, bias = _f32(scale), _f32(bias)
    n, _, _, c = img.shape
    out, d = _alloc_dst(n, c, out_h, out_w, layout, dtype)
    s = _src(img)
    lib().orc_crop_mirror_normalize(C.byref(s), _p(crop_xywh), _p(scale), _p(bias), _p(mirror), _p(vflip),
                                    C.byref(d), C.c_uint(flags))
    return out


def resize(img, roi_xywh, dst_w, dst_h, out_hmax, out_wmax, interp=LINEAR, mirror=None, scale=None, bias=None,
           layout=NHWC, dtype=UINT8, flags=0):
    roi_xywh, dst_w, dst_h, mirror = _u32(roi_xywh), _u32(dst_w), _u32(dst_h), _u32(mirror)
    scale, bias = _f32(scale), _f32(bias)
    n, _, _, c = img.shape
    out, d = _alloc_dst(n, c, out_hmax, out_wmax, layout, dtype)
    s = _src(img)
    lib().orc_resize(C.byref(s), _p(roi_xywh), _p(dst_w), _p(dst_h), C.c_int(interp), _p(mirror), _p(scale),
                     _p(bias), C.byref(d), C.c_uint(flags))
    return out


def _color_common(fn, img, roi_xywh, params, flags, layout=NHWC, dtype=UINT8):
    roi_xywh = _u32(roi_xywh)
    params = [_f32(p) for p in params]
    n, h, w, c = img.shape
    out, d = _alloc_dst(n, c, h, w, layout, dtype)
    s = _src(img)
    fn(C.byref(s), _p(roi_xywh), *[_p(p) for p in params], C.byref(d), C.c_uint(flags))
    return out


def brightness(img, roi_xywh, alpha, beta, flags=0, layout=NHWC, dtype=UINT8):
    return _color_common(lib().orc_brightness, img, roi_xywh, [alpha, beta], flags, layout, dtype)


def contrast(img, roi_xywh, factor, center, flags=0, layout=NHWC, dtype=UINT8):
    return _color_common(lib().orc_contrast, img, roi_xywh, [factor, center], flags, layout, dtype)


def gamma_lut(gamma, flags=0):
    lut = np.empty(256, np.uint8)
    lib().orc_gamma_lut(C.c_float(gamma), _p(lut), C.c_uint(flags))
    return lut


def gamma(img, roi_xywh, gamma, flags=0, layout=NHWC, dtype=UINT8):
    return _color_common(lib().orc_gamma, img, roi_xywh, [gamma], flags, layout, dtype)


def exposure(img, roi_xywh, factor, flags=0, layout=NHWC, dtype=UINT8):
    return _color_common(lib().orc_exposure, img, roi_xywh, [factor], flags, layout, dtype)


def color_temperature(img, roi_xywh, adjustment, flags=0, layout=NHWC, dtype=UINT8):
    roi_xywh = _u32(roi_xywh)
    adj = np.ascontiguousarray(adjustment, np.int32)
    n, h, w, c = img.shape
    out, d = _alloc_dst(n, c, h, w, layout, dtype)
    s = _src(img)
    lib().orc_color_temperature(C.byref(s), _p(roi_xywh), _p(adj), C.byref(d), C.c_uint(flags))
    return out


def normalize(img, roi_xywh, axis_mask=3, mean=None, stddev=None, scale=1.0, shift=0.0, layout=NHWC, dtype=FP32, flags=0):
    roi_xywh = _u32(roi_xywh)
    n, h, w, c = img.shape
    out, d = _alloc_dst(n, c, h, w, layout, dtype)
    s = _src(img)
    m = _f32(mean) if mean is not None else None
    sd = _f32(stddev) if stddev is not None else None
    n_stats = len(m) if m is not None else (len(sd) if sd is not None else 0)
    lib().orc_normalize(C.byref(s), _p(roi_xywh), C.c_uint(axis_mask), _p(m) if m is not None else None, _p(sd) if sd is not None else None,
                        C.c_uint(n_stats), C.c_float(scale), C.c_float(shift), C.byref(d), C.c_uint(flags))
    return out


def blend(img1, img2, roi_xywh, ratio, flags=0, layout=NHWC, dtype=UINT8):
    assert img1.shape == img2.shape
    roi_xywh, ratio = _u32(roi_xywh), _f32(ratio)
    n, h, w, c = img1.shape
    out, d = _alloc_dst(n, c, h, w, layout, dtype)
    s1, s2 = _src(img1), _src(img2)
    lib().orc_blend(C.byref(s1), C.byref(s2), _p(roi_xywh), _p(ratio), C.byref(d), C.c_uint(flags))
    return out


def color_twist(img, roi_xywh, alpha, beta, hue, sat, flags=0, layout=NHWC, dtype=UINT8):
    return _color_common(lib().orc_color_twist, img, roi_xywh, [alpha, beta, hue, sat], flags, layout, dtype)


def warp_affine(img, roi_xywh, affine, dst_w, dst_h, out_hmax, out_wmax, interp=LINEAR, flags=0):
    roi_xywh, dst_w, dst_h = _u32(roi_xywh), _u32(dst_w), _u32(dst_h)
    affine = _f32(affine)
    n, _, _, c = img.shape
    out, d = _alloc_dst(n, c, out_hmax, out_wmax, NHWC, UINT8)
    s = _src(img)
    lib().orc_warp_affine(C.byref(s), _p(roi_xywh), _p(affine), C.c_int(interp), _p(dst_w), _p(dst_h),
                          C.byref(d), C.c_uint(flags))
    return out


def rotate_matrix(angle_deg):
    m = np.empty(6, np.float32)
    lib().orc_rotate_matrix(C.c_float(angle_deg), _p(m))
    return m


def affine_from_rocal(a):
    a = _f32(a)
    m = np.empty(6, np.float32)
    lib().orc_affine_from_rocal(_p(a), _p(m))
    return m


def to_tensor(img, mul, add, reverse_channels=False, layout=NCHW, dtype=FP32, flags=0):
    n, h, w, c = img.shape
    mul, add = _f32(mul), _f32(add)
    out, d = _alloc_dst(n, c, h, w, layout, dtype)
    lib().orc_to_tensor(_p(img), n, h, w, c, _p(mul), _p(add), int(bool(reverse_channels)), C.byref(d),
                        C.c_uint(flags))
    return out


class MT19937:
    def __init__(self, seed):
        self.g = _MT()
        lib().orc_mt19937_seed(C.byref(self.g), C.c_uint32(seed & 0xFFFFFFFF))

    def next(self):
        return int(lib().orc_mt19937_next(C.byref(self.g)))

    def uniform_f32(self, start, end):
        return float(lib().orc_uniform_rand_f32(C.byref(self.g), start, end))

    def uniform_i32(self, start, end):
        return int(lib().orc_uniform_rand_i32(C.byref(self.g), start, end))

    def custom_index(self, freq):
        freq = np.ascontiguousarray(freq, dtype=np.float64)
        return int(lib().orc_custom_rand_index(C.byref(self.g), _p(freq), len(freq)))


def seed_seq_generate(seeds, n):
    seeds = _u32(seeds)
    out = np.empty(n, np.uint32)
    lib().orc_seed_seq_generate(_p(seeds), len(seeds), _p(out), n)
    return out


def fixed_crop(roi_w, roi_h, crop_w, crop_h, anchor=None, x1=0, y1=0):
    out = np.empty(4, np.uint32)
    ax, ay = (anchor if anchor is not None else (0.0, 0.0))
    lib().orc_fixed_crop(roi_w, roi_h, crop_w, crop_h, int(anchor is not None), ax, ay, x1, y1, _p(out))
    return out


class _FParam(C.Structure):
    _fields_ = [("g", _MT), ("lo", C.c_float), ("hi", C.c_float), ("simple", C.c_int), ("value", C.c_float)]


class FParam:
    """A float parameter as the crop laws see it: FParam.uniform(lo, hi, seed) is a UniformRand<float>
    (its constructor draws once), FParam.simple(v) a SimpleParameter<float>."""

    def __init__(self):
        self.p = _FParam()

    @classmethod
    def uniform(cls, lo, hi, seed):
        o = cls()
        lib().orc_fparam_uniform(C.byref(o.p), C.c_float(lo), C.c_float(hi), C.c_uint32(seed & 0xFFFFFFFF))
        return o

    @classmethod
    def simple(cls, v):
        o = cls()
        lib().orc_fparam_simple(C.byref(o.p), C.c_float(v))
        return o

    def renew(self):
        lib().orc_fparam_renew.restype = C.c_float
        return float(lib().orc_fparam_renew(C.byref(self.p)))

    @property
    def value(self):
        return float(self.p.value)


def random_crop(area, aspect, x_drift, y_drift, roi_w, roi_h):
    out = np.empty(4, np.uint32)
    lib().orc_random_crop(C.byref(area.p), C.byref(aspect.p), C.byref(x_drift.p), C.byref(y_drift.p), C.c_uint32(roi_w), C.c_uint32(roi_h), _p(out))
    return out


def factor_crop(h_factor, w_factor, x_drift, y_drift, roi_w, roi_h):
    out = np.empty(4, np.uint32)
    lib().orc_factor_crop(C.byref(h_factor.p), C.byref(w_factor.p), C.byref(x_drift.p), C.byref(y_drift.p), C.c_uint32(roi_w), C.c_uint32(roi_h), _p(out))
    return out


def resize_out_size(sw, sh, dw, dh, mode=0, max_w=0, max_h=0):
    ow, oh = C.c_uint(0), C.c_uint(0)
    lib().orc_resize_out_size(sw, sh, dw, dh, mode, max_w, max_h, C.byref(ow), C.byref(oh))
    return ow.value, oh.value


def num_threads():
    return int(lib().orc_num_threads())
