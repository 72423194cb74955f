"""The augmentation functions of the Python API for the hot-path operators: the reference's names, keyword arguments and defaults
(rocAL_pybind/amd/rocal/fn.py), restated from its text. Each one turns plain numbers into parameter objects where the reference
does, and calls the backend with the arguments in the order of the C entry point (the reference binds the C functions
themselves, rocal_pybind.cpp:1072-1135). Called inside `with pipeline:`."""
from . import types
from .pipeline import Pipeline, b


def _handle():
    if Pipeline._current_pipeline is None:
        raise RuntimeError("fn.* must be called inside `with pipeline:`")
    return Pipeline._current_pipeline._handle


def _fparam(v):
    return b.createFloatParameter(v) if isinstance(v, float) else v


def _iparam(v):
    return b.createIntParameter(v) if isinstance(v, int) else v


def _mirror(mirror):
    # fn.py:563-567, 760-764: an int becomes a fixed 0 / 1 parameter, anything else is a parameter handle already
    if isinstance(mirror, int):
        return b.createIntParameter(0) if mirror == 0 else b.createIntParameter(1)
    return mirror


# ---- fn.py:140-183
def brightness(*inputs, brightness=None, brightness_shift=None, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    """brightness -> alpha (multiplier), brightness_shift -> beta; None draws from the node's default range."""
    return b.brightness(_handle(), inputs[0], False, _fparam(brightness), _fparam(brightness_shift), output_layout, output_dtype)


def brightness_fixed(*inputs, brightness=1.0, brightness_shift=0.0, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    # (the reference hands is_output over in alpha's place, fn.py:171-176; here the values go where the C entry point takes them)
    return b.brightnessFixed(_handle(), inputs[0], float(brightness), float(brightness_shift), False, output_layout, output_dtype)


# ---- fn.py:240-262
def contrast(*inputs, contrast=None, contrast_center=None, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.contrast(_handle(), inputs[0], False, _fparam(contrast), _fparam(contrast_center), output_layout, output_dtype)


# ---- fn.py:265-288
def flip(*inputs, horizontal=0, vertical=0, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.flip(_handle(), inputs[0], False, _iparam(horizontal), _iparam(vertical), output_layout, output_dtype)


# ---- fn.py:291-308
def gamma_correction(*inputs, gamma=0.5, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.gammaCorrection(_handle(), inputs[0], False, _fparam(gamma), output_layout, output_dtype)


# ---- fn.py:311-330
def hue(*inputs, hue=None, device=None, seed=0, output_layout=types.NHWC, output_dtype=types.UINT8):
    """hue change in degrees."""
    return b.hue(_handle(), inputs[0], False, _fparam(hue), output_layout, output_dtype)


# ---- fn.py:625-645
def saturation(*inputs, saturation=1.0, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.saturation(_handle(), inputs[0], False, _fparam(saturation), output_layout, output_dtype)


# ---- fn.py:857-885
def color_twist(*inputs, brightness=1.0, contrast=1.0, hue=0.0, saturation=1.0, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    """brightness -> alpha, contrast -> beta (added on the 0..255 scale), hue in degrees, saturation."""
    return b.colorTwist(_handle(), inputs[0], False, _fparam(brightness), _fparam(contrast), _fparam(hue), _fparam(saturation), output_layout, output_dtype)


# ---- fn.py:400-424
def resize(*inputs, max_size=[], resize_longer=0, resize_shorter=0, resize_width=0, resize_height=0, scaling_mode=types.SCALING_MODE_DEFAULT,
           interpolation_type=types.LINEAR_INTERPOLATION, antialias=True, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.resize(_handle(), inputs[0], resize_width, resize_height, False, scaling_mode, max_size, resize_shorter, resize_longer,
                    interpolation_type, output_layout, output_dtype)


# ---- fn.py:427-460
def resize_crop_mirror(*inputs, resize_width=0, resize_height=0, crop_w=0, crop_h=0, mirror=1, device=None, max_size=[], resize_longer=0,
                       resize_shorter=0, scaling_mode=types.SCALING_MODE_DEFAULT, interpolation_type=types.LINEAR_INTERPOLATION,
                       output_layout=types.NHWC, output_dtype=types.UINT8):
    # (the C entry point takes crop_h before crop_w, rocal_api_augmentation.h:1022; the values go where it takes them)
    return b.resizeCropMirrorFixed(_handle(), inputs[0], resize_width, resize_height, False, crop_h, crop_w, _mirror(mirror), output_layout, output_dtype)


# ---- fn.py:463-500
def resize_crop(*inputs, resize_width=0, resize_height=0, crop_area_factor=None, crop_aspect_ratio=None, x_drift=None, y_drift=None, device=None,
                max_size=[], resize_longer=0, resize_shorter=0, scaling_mode=types.SCALING_MODE_DEFAULT,
                interpolation_type=types.LINEAR_INTERPOLATION, output_layout=types.NHWC, output_dtype=types.UINT8):
    """The random-resized-crop node (rocalCropResize): a window drawn from area factor / aspect ratio / drifts, resized."""
    return b.cropResize(_handle(), inputs[0], resize_width, resize_height, False, _fparam(crop_area_factor), _fparam(crop_aspect_ratio),
                        _fparam(x_drift), _fparam(y_drift), output_layout, output_dtype)


random_resized_crop = resize_crop


# ---- fn.py:503-526
def roi_resize(*inputs, resize_width=0, resize_height=0, roi_w=None, roi_h=None, roi_pos_x=None, roi_pos_y=None, device=None,
               interpolation_type=types.LINEAR_INTERPOLATION, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.roiResize(_handle(), inputs[0], resize_width, resize_height, False, roi_h, roi_w, roi_pos_x, roi_pos_y, interpolation_type,
                       output_layout, output_dtype)


# ---- fn.py:529-569
def resize_mirror_normalize(*inputs, max_size=[], resize_longer=0, resize_shorter=0, resize_width=0, resize_height=0,
                            scaling_mode=types.SCALING_MODE_DEFAULT, interpolation_type=types.LINEAR_INTERPOLATION, mean=[0.0], std=[1.0], mirror=1,
                            device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.resizeMirrorNormalize(_handle(), inputs[0], resize_width, resize_height, mean, std, False, scaling_mode, max_size, resize_shorter,
                                   resize_longer, interpolation_type, _mirror(mirror), output_layout, output_dtype)


# ---- fn.py:572-596
def random_crop(*inputs, crop_area_factor=[0.08, 1], crop_aspect_ratio=[0.75, 1.333333], crop_pox_x=0, crop_pox_y=0, num_attempts=20, device=None,
                all_boxes_above_threshold=True, allow_no_crop=True, ltrb=True, output_layout=types.NHWC, output_dtype=types.UINT8):
    """Ranges [lo, hi] become uniform random parameters; positions 0 leave the node's default (random) drifts."""
    def rng(v):
        if isinstance(v, (list, tuple)):
            return b.createFloatUniformRand(float(v[0]), float(v[1]))
        return _fparam(v) if isinstance(v, float) else (None if v == 0 else v)
    return b.randomCrop(_handle(), inputs[0], False, rng(crop_area_factor), rng(crop_aspect_ratio), rng(crop_pox_x), rng(crop_pox_y), num_attempts,
                        output_layout, output_dtype)


# ---- fn.py:599-622
def rotate(*inputs, angle=None, dest_width=0, dest_height=0, interpolation_type=types.LINEAR_INTERPOLATION, device=None, fill_value=None,
           output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.rotate(_handle(), inputs[0], False, _fparam(angle), dest_width, dest_height, interpolation_type, output_layout, output_dtype)


# ---- fn.py:686-707
def warp_affine(*inputs, dest_width=0, dest_height=0, matrix=[0, 0, 0, 0, 0, 0], interpolation_type=types.LINEAR_INTERPOLATION, device=None,
                output_layout=types.NHWC, output_dtype=types.UINT8):
    """matrix = [x0, x1, y0, y1, o0, o1]: source = [[x0, x1, o0], [y0, y1, o1]] applied to the destination about the centres."""
    x0, x1, y0, y1, o0, o1 = matrix
    return b.warpAffineFixed(_handle(), inputs[0], float(x0), float(x1), float(y0), float(y1), float(o0), float(o1), False, dest_height, dest_width,
                             interpolation_type, output_layout, output_dtype)


def _crop_dims(crop, crop_h, crop_w, crop_d=1):
    # fn.py:749-758, 787-798: [h, w], [d, h, w] or the separate keywords
    if len(crop) == 2:
        return crop_d, crop[0], crop[1]
    if len(crop) == 3:
        return crop[0], crop[1], crop[2]
    return crop_d, crop_h, crop_w


# ---- fn.py:731-771
def crop_mirror_normalize(*inputs, crop=[0, 0], crop_pos_x=0.5, crop_pos_y=0.5, crop_w=0, crop_h=0, mean=[0.0], std=[1.0], mirror=1, device=None,
                          output_layout=types.NHWC, output_dtype=types.UINT8):
    _, crop_height, crop_width = _crop_dims(crop, crop_h, crop_w)
    return b.cropMirrorNormalize(_handle(), inputs[0], crop_height, crop_width, crop_pos_x, crop_pos_y, mean, std, False, _mirror(mirror),
                                 output_layout, output_dtype)


# ---- fn.py:774-806
def center_crop(*inputs, crop=[0, 0], crop_h=0, crop_w=0, crop_d=1, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    crop_depth, crop_height, crop_width = _crop_dims(crop, crop_h, crop_w, crop_d)
    return b.centerCropFixed(_handle(), inputs[0], crop_width, crop_height, crop_depth, False, output_layout, output_dtype)


# ---- fn.py:809-854
def crop(*inputs, crop=[0, 0], crop_pos_x=0.5, crop_pos_y=0.5, crop_pos_z=0.5, crop_w=0, crop_h=0, crop_d=1, device=None,
         output_layout=types.NHWC, output_dtype=types.UINT8):
    crop_depth, crop_height, crop_width = _crop_dims(crop, crop_h, crop_w, crop_d)
    if crop_width == 0 and crop_height == 0:  # no size given: the random crop node with its default ranges
        return b.crop(_handle(), inputs[0], False, None, None, None, None, None, None, output_layout, output_dtype)
    return b.cropFixed(_handle(), inputs[0], crop_width, crop_height, crop_depth, False, float(crop_pos_x), float(crop_pos_y), float(crop_pos_z),
                       output_layout, output_dtype)


# ---- the streaming neighbours (fn.py: exposure, color_temp, blend)
def exposure(*inputs, exposure=0.5, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.exposure(_handle(), inputs[0], False, _fparam(exposure), output_layout, output_dtype)


def color_temp(*inputs, adjustment_value=50, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.colorTemp(_handle(), inputs[0], False, _iparam(adjustment_value), output_layout, output_dtype)


def blend(*inputs, ratio=None, device=None, output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.blend(_handle(), inputs[0], inputs[1], False, _fparam(ratio), output_layout, output_dtype)


# ---- fn.py: normalize (axes, mean, stddev, scale, shift) and transpose (perm) on image tensors
def normalize(*inputs, axes=[], mean=[], stddev=[], scale=1.0, shift=0.0, output_datatype=types.FLOAT, output_dtype=None):
    """axes: the reduced axes (0 height, 1 width, 2 channels); empty mean / stddev are computed per sample.
    The keyword is `output_datatype` as in the reference (rocAL_pybind/amd/rocal/fn.py:1216); `output_dtype`, the spelling of
    every other operator, is accepted as well."""
    return b.normalize(_handle(), inputs[0], axes, mean, stddev, False, scale, shift, output_datatype if output_dtype is None else output_dtype)


def transpose(*inputs, perm=[], output_layout=types.NHWC, output_dtype=types.UINT8):
    return b.transpose(_handle(), inputs[0], perm, False, output_layout)
