"""Loader for the C-ABI shared library (rocal_amd/lib/librocal_mi355x.so).

There is no CPU fallback: if the HIP library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("RMX_LIB", os.path.join(_HERE, "lib", "librocal_mi355x.so"))


class TensorDesc(C.Structure):
    """Mirror of rmx_tensor_desc (include/rocal_mi355x.h)."""
    _fields_ = [("n", C.c_uint32), ("h", C.c_uint32), ("w", C.c_uint32), ("c", C.c_uint32),
                ("layout", C.c_int32), ("dtype", C.c_int32)]


class RmxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("rocal_mi355x error %d: %s" % (code, msg))
        self.code = code


_lib = None
_vp = C.c_void_p

# name -> argtypes ; every function returns int unless listed in _RESTYPES
_SIGS = {
    "rmx_ctx_create": [C.c_int, _vp, C.c_int, C.POINTER(_vp)],
    "rmx_ctx_destroy": [_vp],
    "rmx_ctx_sync": [_vp],
    "rmx_ctx_stream": [_vp],
    "rmx_last_error": [],
    "rmx_version": [],
    "rmx_op_launch": [_vp, _vp, _vp],
    "rmx_op_destroy": [_vp],
    "rmx_op_algorithmic_bytes": [_vp],
    "rmx_op_kernel_name": [_vp],
    "rmx_op_plan": [_vp],
    "rmx_op_set_ragged_source": [_vp, _vp, _vp, _vp, C.c_uint64],
    "rmx_op_set_ragged_source_strided": [_vp, _vp, _vp, _vp, _vp, C.c_uint64],
    "rmx_create_crop_mirror_normalize": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_crop_mirror_normalize": [_vp, _vp, _vp, _vp, _vp],
    "rmx_create_crop": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_crop": [_vp, _vp],
    "rmx_create_flip": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_flip": [_vp, _vp, _vp, _vp],
    "rmx_create_resize": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.c_int, C.c_uint32, C.POINTER(_vp)],
    "rmx_update_resize": [_vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "rmx_update_resize_cmn": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "rmx_update_resize_color_cmn": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
    "rmx_create_color_twist": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_color_twist": [_vp, _vp, _vp, _vp, _vp, _vp],
    "rmx_create_brightness": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_brightness": [_vp, _vp, _vp, _vp],
    "rmx_create_contrast": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_contrast": [_vp, _vp, _vp, _vp],
    "rmx_create_hue": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_hue": [_vp, _vp, _vp],
    "rmx_create_saturation": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_saturation": [_vp, _vp, _vp],
    "rmx_create_gamma": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_gamma": [_vp, _vp, _vp],
    "rmx_create_exposure": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_exposure": [_vp, _vp, _vp],
    "rmx_create_color_temperature": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_color_temperature": [_vp, _vp, _vp],
    "rmx_create_blend": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_blend": [_vp, _vp, _vp],
    "rmx_op_launch2": [_vp, _vp, _vp, _vp],
    "rmx_create_warp_affine": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.c_int, C.POINTER(_vp)],
    "rmx_update_warp_affine": [_vp, _vp, _vp, _vp, _vp],
    "rmx_create_rotate": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.c_int, C.POINTER(_vp)],
    "rmx_update_rotate": [_vp, _vp, _vp, _vp, _vp],
    "rmx_create_to_tensor": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.POINTER(_vp)],
    "rmx_update_to_tensor": [_vp, _vp, _vp, C.c_int],
    "rmx_create_normalize": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.POINTER(_vp)],
    "rmx_update_normalize": [_vp, _vp, C.c_uint32, _vp, _vp, C.c_uint32, C.c_float, C.c_float],
    "rmx_create_transpose": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), _vp, C.c_int, C.POINTER(_vp)],
    "rmx_update_transpose": [_vp, _vp],
    "rmx_copy_bytes": [_vp, _vp, _vp, C.c_size_t],
    "rmx_stream_probe": [_vp, C.c_int, _vp, _vp, C.c_size_t, C.c_int],
    "rmx_resize_cmn_noalloc": [_vp, C.POINTER(TensorDesc), C.POINTER(TensorDesc), C.c_int, C.c_int, C.c_uint32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp],
}
_RESTYPES = {"rmx_last_error": C.c_char_p, "rmx_version": C.c_char_p, "rmx_ctx_stream": _vp,
             "rmx_op_algorithmic_bytes": C.c_uint64, "rmx_op_kernel_name": C.c_char_p, "rmx_op_plan": C.c_char_p}

EXPORTS = tuple(_SIGS)


def lib():
    """Load the library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RmxError(-1, "HIP library not built: %s is missing (run `python -m rocal_amd.build`)" % LIB_PATH)
        # PyTorch bundles its own HIP runtime; load it first so that this library binds to the same
        # runtime instance (two instances in one process do not see each other's devices/streams).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        l = C.CDLL(LIB_PATH)
        for name, args in _SIGS.items():
            fn = getattr(l, name)
            fn.argtypes = args
            fn.restype = _RESTYPES.get(name, C.c_int)
        _lib = l
    return _lib


def check(code):
    if code != 0:
        raise RmxError(code, lib().rmx_last_error().decode())
