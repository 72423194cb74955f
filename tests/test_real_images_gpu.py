"""Natural pixels through the rocal* entry points: eight 299 x 299 images of the reference's own test data
(tests/golden/amd_tiny_8.npz, decoded from data/images/AMD-tinyDataSet by tests/golden/make_real_images.py) run through the
fixed-parameter cases of the reference's unit tests (tests/cpp_api/unit_tests/unit_tests.cpp:605-624,730-735,745-856:
Resize 400 x 400 bilinear and triangular, CropMirrorNormalize 224 x 224 with mean 128 and std 1.2, RotateFixed 45,
WarpAffineFixed(1,1,.5,.5,7,7), ResizeCropMirrorFixed 400 -> 200, ColorTwistFixed(.2,10,100,.25) and the other point and
crop cases), built by the C++ driver through include/rocal_api_mi355x.h, against the oracle. 299-pixel rows (897 bytes: odd
widths, rows at every byte phase) take the any-width and general forms of the kernels on natural content. The reference's
golden PNGs for these cases live in an external data repository, so this checks kernels against oracle on the reference's
inputs, not against RPP's outputs."""
import os
import subprocess

import numpy as np
import pytest

from oracle import orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_CHECK = os.path.join(ROOT, "rocal_amd", "lib", "host_check")
N, S = 8, 299


def _same(got, exp, what):
    assert got.shape == exp.shape, what
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "%s: %d values differ" % (what, int((got != exp).sum()))


def test_reference_unit_test_cases_on_the_reference_images(tmp_path):
    data = np.load(os.path.join(ROOT, "tests", "golden", "amd_tiny_8.npz"), allow_pickle=False)
    img = np.ascontiguousarray(data["images"])
    assert img.shape == (N, S, S, 3) and img.dtype == np.uint8
    img.tofile(tmp_path / "input.bin")
    with open(tmp_path / "meta.txt", "w") as f:
        f.write("%d %d %d\n" % (N, S, S) + "%d %d\n" % (S, S) * N)
    print("host_check pipeline ref_cases", flush=True)
    p = subprocess.run([HOST_CHECK, "pipeline", "ref_cases", str(tmp_path)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, (p.returncode, p.stdout, p.stderr[-3000:])
    u8 = np.uint8
    shapes = [(400, 400), (400, 400), (224, 224), (224, 224), (224, 224), (S, S), (S, S), (S, S), (S, S), (S, S), (S, S), (S, S), (S, S), (S, S),
              (S, S), (S, S), (S, S), (224, 224), (224, 224), (400, 400), (400, 400)]
    outs = [np.fromfile(tmp_path / ("out%d_b1.bin" % k), dtype=u8).reshape(N, h, w, 3) for k, (h, w) in enumerate(shapes)]
    full = np.array([[0, 0, S, S]] * N, np.uint32)
    one = lambda v: np.full(N, v, np.float32)
    ones = np.ones(N, np.uint32)
    d400 = np.full(N, 400, np.uint32)
    scale, bias = orc.cmn_scale_bias([128, 128, 128], [1.2, 1.2, 1.2], N)
    k = iter(range(len(shapes)))
    _same(outs[next(k)], orc.resize(img, full, d400, d400, 400, 400, interp=orc.LINEAR), "Resize 400 x 400 bilinear")
    _same(outs[next(k)], orc.resize(img, full, d400, d400, 400, 400, interp=orc.TRIANGULAR), "Resize 400 x 400 triangular")
    corner = np.stack([orc.fixed_crop(S, S, 224, 224, anchor=(0.0, 0.0))] * N)
    _same(outs[next(k)], orc.crop_mirror_normalize(img, corner, scale, bias, ones, 224, 224, orc.NHWC, orc.UINT8), "CropMirrorNormalize at (0, 0)")
    centre = np.stack([orc.fixed_crop(S, S, 224, 224, anchor=(0.5, 0.5))] * N)
    _same(outs[next(k)], orc.crop_mirror_normalize(img, centre, scale, bias, ones, 224, 224, orc.NHWC, orc.UINT8), "CropMirrorNormalize, centre")
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.25), s(1.2), s(0.6), s(0.4), S, S)] * N)
    d224 = np.full(N, 224, np.uint32)
    _same(outs[next(k)], orc.resize(img, window, d224, d224, 224, 224, interp=orc.LINEAR), "CropResizeFixed(0.25, 1.2, 0.6, 0.4)")
    dS = np.full(N, S, np.uint32)
    rot = orc.warp_affine(img, full, np.stack([orc.rotate_matrix(45.0)] * N), dS, dS, S, S, interp=orc.LINEAR)
    _same(outs[next(k)], rot, "RotateFixed 45")
    _same(outs[next(k)], orc.brightness(img, full, one(1.90), one(20.0)), "BrightnessFixed(1.9, 20)")
    _same(outs[next(k)], orc.gamma(img, full, one(0.5)), "GammaFixed 0.5")
    _same(outs[next(k)], orc.contrast(img, full, one(30.0), one(80.0)), "ContrastFixed(30, 80)")
    _same(outs[next(k)], orc.blend(img, rot, full, one(0.5)), "BlendFixed(source, rotated, 0.5)")
    m = np.stack([orc.affine_from_rocal([1, 0.5, 1, 0.5, 7, 7])] * N)  # x0, y0, x1, y1, o0, o1 of WarpAffineFixed(x0=1, x1=1, y0=.5, y1=.5, o0=7, o1=7)
    _same(outs[next(k)], orc.warp_affine(img, full, m, dS, dS, S, S, interp=orc.LINEAR), "WarpAffineFixed(1, 1, .5, .5, 7, 7)")
    _same(outs[next(k)], orc.color_temperature(img, full, np.full(N, 70, np.int32)), "ColorTempFixed 70")
    _same(outs[next(k)], orc.exposure(img, full, one(1.0)), "ExposureFixed 1")
    _same(outs[next(k)], orc.crop_mirror_normalize(img, full, None, None, ones, S, S, orc.NHWC, orc.UINT8, vflip=np.zeros(N, np.uint32)), "FlipFixed(1, 0)")
    _same(outs[next(k)], orc.color_twist(img, full, one(1.0), one(0.0), one(150.0), one(1.0)), "HueFixed 150")
    _same(outs[next(k)], orc.color_twist(img, full, one(1.0), one(0.0), one(0.0), one(0.3)), "SaturationFixed 0.3")
    _same(outs[next(k)], orc.color_twist(img, full, one(0.2), one(10.0), one(100.0), one(0.25)), "ColorTwistFixed(.2, 10, 100, .25)")
    _same(outs[next(k)], orc.crop_mirror_normalize(img, corner, None, None, None, 224, 224, orc.NHWC, orc.UINT8), "CropFixed 224 x 224 at the origin")
    _same(outs[next(k)], orc.crop_mirror_normalize(img, centre, None, None, None, 224, 224, orc.NHWC, orc.UINT8), "CropCenterFixed 224 x 224")
    w200 = np.stack([orc.fixed_crop(S, S, 200, 200)] * N)
    _same(outs[next(k)], orc.resize(img, w200, d400, d400, 400, 400, interp=orc.LINEAR, mirror=ones), "ResizeCropMirrorFixed(400, 400, 200, 200)")
    _same(outs[next(k)], orc.resize(img, full, d400, d400, 400, 400, interp=orc.LINEAR, mirror=ones, scale=scale, bias=bias, layout=orc.NHWC,
                                    dtype=orc.UINT8), "ResizeMirrorNormalize 400 x 400")
