"""Constants of the Python API with the reference's names and values (rocAL_pybind/amd/rocal/types.py, which re-exports the
enums of rocAL/include/api/rocal_api_types.h)."""
# RocalStatus
OK, CONTEXT_INVALID, RUNTIME_ERROR, UPDATE_PARAMETER_FAILED, INVALID_PARAMETER_TYPE = 0, 1, 2, 3, 4
# RocalProcessMode
GPU, CPU = 0, 1
# RocalTensorOutputType
FLOAT, FLOAT16, UINT8 = 0, 1, 2
# RocalTensorLayout
NHWC, NCHW, NONE = 0, 1, 9
# RocalOutputMemType
HOST_MEMORY, DEVICE_MEMORY, PINNED_MEMORY = 0, 1, 2
# RocalResizeScalingMode
SCALING_MODE_DEFAULT, SCALING_MODE_STRETCH, SCALING_MODE_NOT_SMALLER, SCALING_MODE_NOT_LARGER, SCALING_MODE_MIN_MAX = 0, 1, 2, 3, 4
# RocalResizeInterpolationType
(NEAREST_NEIGHBOR_INTERPOLATION, LINEAR_INTERPOLATION, CUBIC_INTERPOLATION, LANCZOS_INTERPOLATION, GAUSSIAN_INTERPOLATION,
 TRIANGULAR_INTERPOLATION) = 0, 1, 2, 3, 4, 5
