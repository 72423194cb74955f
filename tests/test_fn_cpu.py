"""The Python fn.* layer without a GPU: every keyword's default and renaming is checked against the positional arguments that
reach the backend (= the C entry point's order, rocAL/include/api/rocal_api_augmentation.h). Expected tuples are written out
by hand from the reference's headers and fn.py text."""
import pytest

from rocal_amd import fn, pipeline, types


class Recorder:
    """Stands for the backend: parameters become tagged tuples, augmentation calls are recorded."""

    def __init__(self):
        self.calls = []

    def createFloatParameter(self, v):
        return ("F", v)

    def createIntParameter(self, v):
        return ("I", v)

    def createFloatUniformRand(self, a, b_):
        return ("FU", a, b_)

    def __getattr__(self, name):
        def call(*args):
            self.calls.append((name,) + args)
            return ("T", name)
        return call


class _Pipe:
    _handle = "H"


@pytest.fixture
def rec(monkeypatch):
    r = Recorder()
    monkeypatch.setattr(fn, "b", r)
    monkeypatch.setattr(pipeline.Pipeline, "_current_pipeline", _Pipe())
    return r


U8, NHWC = types.UINT8, types.NHWC


def test_crop_mirror_normalize_defaults_and_keywords(rec):
    fn.crop_mirror_normalize("in")
    # crop=[0,0] -> height 0, width 0; crop_pos 0.5; mean [0.0], std [1.0]; mirror=1 -> IntParameter(1); NHWC, UINT8
    assert rec.calls[-1] == ("cropMirrorNormalize", "H", "in", 0, 0, 0.5, 0.5, [0.0], [1.0], False, ("I", 1), NHWC, U8)
    fn.crop_mirror_normalize("in", crop=(224, 200), mirror=0, mean=[1, 2, 3], std=[4, 5, 6], output_layout=types.NCHW, output_dtype=types.FLOAT16)
    assert rec.calls[-1] == ("cropMirrorNormalize", "H", "in", 224, 200, 0.5, 0.5, [1, 2, 3], [4, 5, 6], False, ("I", 0), types.NCHW, types.FLOAT16)
    fn.crop_mirror_normalize("in", crop=(1, 30, 40), crop_pos_x=0.25, crop_pos_y=0.75, mirror="coin")  # [d, h, w]; a parameter handle passes through
    assert rec.calls[-1][3:7] == (30, 40, 0.25, 0.75) and rec.calls[-1][10] == "coin"
    fn.crop_mirror_normalize("in", crop=[], crop_h=7, crop_w=9, mirror=5)  # any non-zero int is a fixed 1
    assert rec.calls[-1][3:5] == (7, 9) and rec.calls[-1][10] == ("I", 1)


def test_resize_family(rec):
    fn.resize("in")
    # dest_width, dest_height, is_output, scaling_mode DEFAULT(0), max_size [], shorter, longer, LINEAR
    assert rec.calls[-1] == ("resize", "H", "in", 0, 0, False, types.SCALING_MODE_DEFAULT, [], 0, 0, types.LINEAR_INTERPOLATION, NHWC, U8)
    fn.resize("in", resize_width=640, resize_height=360, interpolation_type=types.TRIANGULAR_INTERPOLATION, resize_shorter=3, resize_longer=4, max_size=[9, 8],
              scaling_mode=types.SCALING_MODE_NOT_SMALLER)
    assert rec.calls[-1] == ("resize", "H", "in", 640, 360, False, types.SCALING_MODE_NOT_SMALLER, [9, 8], 3, 4, types.TRIANGULAR_INTERPOLATION, NHWC, U8)
    fn.resize_crop("in", resize_width=224, resize_height=224, crop_area_factor=0.5, x_drift=0.25)
    assert rec.calls[-1] == ("cropResize", "H", "in", 224, 224, False, ("F", 0.5), None, ("F", 0.25), None, NHWC, U8)
    assert fn.random_resized_crop is fn.resize_crop
    fn.resize_mirror_normalize("in", resize_width=10, resize_height=20)
    assert rec.calls[-1] == ("resizeMirrorNormalize", "H", "in", 10, 20, [0.0], [1.0], False, types.SCALING_MODE_DEFAULT, [], 0, 0,
                             types.LINEAR_INTERPOLATION, ("I", 1), NHWC, U8)
    fn.resize_crop_mirror("in", resize_width=36, resize_height=28, crop_w=50, crop_h=40, mirror=0)
    assert rec.calls[-1] == ("resizeCropMirrorFixed", "H", "in", 36, 28, False, 40, 50, ("I", 0), NHWC, U8)  # crop_h before crop_w
    fn.roi_resize("in", resize_width=5, resize_height=6, roi_w=7, roi_h=8, roi_pos_x=0.1, roi_pos_y=0.2)
    assert rec.calls[-1] == ("roiResize", "H", "in", 5, 6, False, 8, 7, 0.1, 0.2, types.LINEAR_INTERPOLATION, NHWC, U8)  # roi_h before roi_w


def test_colour_family_renamings(rec):
    fn.color_twist("in")
    # brightness -> alpha, contrast -> beta, hue, saturation; defaults 1.0, 1.0, 0.0, 1.0 become fixed parameters
    assert rec.calls[-1] == ("colorTwist", "H", "in", False, ("F", 1.0), ("F", 1.0), ("F", 0.0), ("F", 1.0), NHWC, U8)
    fn.color_twist("in", brightness=1.2, contrast=8.0, hue=40.0, saturation=1.3)
    assert rec.calls[-1][4:8] == (("F", 1.2), ("F", 8.0), ("F", 40.0), ("F", 1.3))
    fn.brightness("in")
    assert rec.calls[-1] == ("brightness", "H", "in", False, None, None, NHWC, U8)  # None: the node's default random range
    fn.brightness("in", brightness=0.5, brightness_shift=100.0)
    assert rec.calls[-1][4:6] == (("F", 0.5), ("F", 100.0))  # brightness -> alpha, brightness_shift -> beta
    fn.brightness_fixed("in")
    assert rec.calls[-1] == ("brightnessFixed", "H", "in", 1.0, 0.0, False, NHWC, U8)
    fn.contrast("in", contrast=1.4, contrast_center=100.0)
    assert rec.calls[-1] == ("contrast", "H", "in", False, ("F", 1.4), ("F", 100.0), NHWC, U8)
    fn.hue("in", hue=30.0)
    assert rec.calls[-1] == ("hue", "H", "in", False, ("F", 30.0), NHWC, U8)
    fn.saturation("in")
    assert rec.calls[-1] == ("saturation", "H", "in", False, ("F", 1.0), NHWC, U8)
    fn.gamma_correction("in")
    assert rec.calls[-1] == ("gammaCorrection", "H", "in", False, ("F", 0.5), NHWC, U8)
    fn.exposure("in")
    assert rec.calls[-1] == ("exposure", "H", "in", False, ("F", 0.5), NHWC, U8)
    fn.color_temp("in")
    assert rec.calls[-1] == ("colorTemp", "H", "in", False, ("I", 50), NHWC, U8)
    fn.blend("a", "b", ratio=0.3)
    assert rec.calls[-1] == ("blend", "H", "a", "b", False, ("F", 0.3), NHWC, U8)


def test_flip_warp_rotate_crop(rec):
    fn.flip("in")
    assert rec.calls[-1] == ("flip", "H", "in", False, ("I", 0), ("I", 0), NHWC, U8)  # ints become IntParameters
    fn.flip("in", horizontal=1, vertical="p")
    assert rec.calls[-1][4:6] == (("I", 1), "p")
    fn.warp_affine("in", dest_width=48, dest_height=56, matrix=[1.05, 0.1, -0.08, 0.95, 3.0, -2.0])
    # matrix = [x0, x1, y0, y1, o0, o1] in that order, then is_output, dest_HEIGHT, dest_WIDTH
    assert rec.calls[-1] == ("warpAffineFixed", "H", "in", 1.05, 0.1, -0.08, 0.95, 3.0, -2.0, False, 56, 48, types.LINEAR_INTERPOLATION, NHWC, U8)
    fn.rotate("in", angle=30.0, dest_width=5, dest_height=6)
    assert rec.calls[-1] == ("rotate", "H", "in", False, ("F", 30.0), 5, 6, types.LINEAR_INTERPOLATION, NHWC, U8)
    fn.rotate("in")
    assert rec.calls[-1][4] is None  # no angle: the node's default random range
    fn.center_crop("in", crop=(24, 32))
    assert rec.calls[-1] == ("centerCropFixed", "H", "in", 32, 24, 1, False, NHWC, U8)  # width before height
    fn.crop("in", crop=(20, 30), crop_pos_x=0.1, crop_pos_y=0.2)
    assert rec.calls[-1] == ("cropFixed", "H", "in", 30, 20, 1, False, 0.1, 0.2, 0.5, NHWC, U8)
    fn.crop("in")
    assert rec.calls[-1] == ("crop", "H", "in", False, None, None, None, None, None, None, NHWC, U8)
    fn.random_crop("in")
    assert rec.calls[-1] == ("randomCrop", "H", "in", False, ("FU", 0.08, 1.0), ("FU", 0.75, 1.333333), None, None, 20, NHWC, U8)


def test_normalize_and_transpose(rec):
    fn.normalize("in")
    assert rec.calls[-1] == ("normalize", "H", "in", [], [], [], False, 1.0, 0.0, types.FLOAT)
    fn.normalize("in", output_datatype=types.FLOAT16)  # the reference's spelling of the keyword (fn.py:1216)
    assert rec.calls[-1] == ("normalize", "H", "in", [], [], [], False, 1.0, 0.0, types.FLOAT16)
    fn.normalize("in", axes=[0, 1], mean=[1.0], stddev=[2.0], scale=3.0, shift=4.0, output_dtype=types.FLOAT16)
    assert rec.calls[-1] == ("normalize", "H", "in", [0, 1], [1.0], [2.0], False, 3.0, 4.0, types.FLOAT16)
    fn.transpose("in", perm=[2, 0, 1], output_layout=types.NCHW)
    assert rec.calls[-1] == ("transpose", "H", "in", [2, 0, 1], False, types.NCHW)


def test_fn_needs_a_current_pipeline(monkeypatch):
    monkeypatch.setattr(pipeline.Pipeline, "_current_pipeline", None)
    with pytest.raises(RuntimeError, match="with pipeline"):
        fn.flip("in")


def test_backend_binds_every_entry_point_it_names():
    """The host library exports every symbol the ctypes backend declares (no call is made)."""
    from rocal_amd import backend
    h = backend.host()
    for name in backend._SIGS:
        assert hasattr(h, name), name
