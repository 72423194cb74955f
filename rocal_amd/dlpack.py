"""DLPack export of a pipeline tensor: the consumer (torch.from_dlpack, cupy, ...) aliases the device buffer the last node wrote,
without a copy. Stands where the reference copies a finished output into the framework's tensor
(rocAL/source/pipeline/tensor.cpp:419-454, rocAL_pybind/amd/rocal/plugin/pytorch.py:118-135). The capsule follows the DLPack
ABI (DLManagedTensor, capsule name "dltensor", device type kDLROCM); the memory belongs to the pipeline, so the consumer's view
is valid until the pipeline writes the tensor again (the next run) or is released."""
import ctypes as C

from . import types

kDLROCM = 10
kDLUInt, kDLFloat = 1, 2


class DLDevice(C.Structure):
    _fields_ = [("device_type", C.c_int32), ("device_id", C.c_int32)]


class DLDataType(C.Structure):
    _fields_ = [("code", C.c_uint8), ("bits", C.c_uint8), ("lanes", C.c_uint16)]


class DLTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("device", DLDevice), ("ndim", C.c_int32), ("dtype", DLDataType), ("shape", C.POINTER(C.c_int64)),
                ("strides", C.POINTER(C.c_int64)), ("byte_offset", C.c_uint64)]


class DLManagedTensor(C.Structure):
    pass


_DELETER = C.CFUNCTYPE(None, C.POINTER(DLManagedTensor))
DLManagedTensor._fields_ = [("dl_tensor", DLTensor), ("manager_ctx", C.c_void_p), ("deleter", _DELETER)]

_alive = {}  # address of a managed tensor -> (struct, shape array, keep-alive object) until the consumer calls the deleter


@_DELETER
def _deleter(p):
    _alive.pop(C.addressof(p.contents), None)


# A capsule that is dropped without having been consumed still carries the name "dltensor": its destructor then calls the
# deleter (the DLPack producer rule); a consumer renames the capsule ("used_dltensor") and calls the deleter itself.
_CAPSULE_DESTRUCTOR = C.CFUNCTYPE(None, C.c_void_p)
_capsule_is_valid = C.pythonapi.PyCapsule_IsValid
_capsule_is_valid.restype = C.c_int
_capsule_is_valid.argtypes = [C.c_void_p, C.c_char_p]
_capsule_get_pointer = C.pythonapi.PyCapsule_GetPointer
_capsule_get_pointer.restype = C.c_void_p
_capsule_get_pointer.argtypes = [C.c_void_p, C.c_char_p]


@_CAPSULE_DESTRUCTOR
def _capsule_destructor(capsule):
    if _capsule_is_valid(capsule, b"dltensor"):
        _alive.pop(_capsule_get_pointer(capsule, b"dltensor"), None)


_capsule_new = C.pythonapi.PyCapsule_New
_capsule_new.restype = C.py_object
_capsule_new.argtypes = [C.c_void_p, C.c_char_p, _CAPSULE_DESTRUCTOR]


def to_dlpack(device_ptr, shape, dtype, device_id=0, keep_alive=None):
    """A "dltensor" capsule for `shape` elements of `dtype` (types.FLOAT / FLOAT16 / UINT8), dense row-major, at `device_ptr`."""
    code, bits = {types.FLOAT: (kDLFloat, 32), types.FLOAT16: (kDLFloat, 16), types.UINT8: (kDLUInt, 8)}[dtype]
    m = DLManagedTensor()
    dims = (C.c_int64 * len(shape))(*[int(d) for d in shape])
    m.dl_tensor.data = device_ptr
    m.dl_tensor.device = DLDevice(kDLROCM, device_id)
    m.dl_tensor.ndim = len(shape)
    m.dl_tensor.dtype = DLDataType(code, bits, 1)
    m.dl_tensor.shape = dims
    m.dl_tensor.strides = None  # dense, row-major
    m.dl_tensor.byte_offset = 0
    m.manager_ctx = None
    m.deleter = _deleter
    _alive[C.addressof(m)] = (m, dims, keep_alive)
    return _capsule_new(C.addressof(m), b"dltensor", _capsule_destructor)
