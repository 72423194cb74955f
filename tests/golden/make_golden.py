"""Writes the small input/output vectors under tests/golden/.

rocAL keeps no numeric vectors for these ops in its tree (its golden PNGs live in an external
data repository, tests/cpp_api/unit_tests/testAllScripts.sh:19-31), and RPP is not available, so
these fixtures are OUTPUTS OF THIS REPOSITORY'S CPU ORACLE on seeded inputs, with the fixed
parameters of the reference's own unit tests (tests/cpp_api/unit_tests/unit_tests.cpp:605-850).
They pin the oracle against drift and let the GPU box check the HIP path without the oracle.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import orc  # noqa: E402
from rocal_amd import workloads as wl  # noqa: E402


def cases():
    rng = np.random.default_rng(4242)
    n, H, W = 2, 48, 64
    img = wl.smooth_noise(rng, n, H, W, sigma=1.5)
    img[1] = rng.integers(0, 256, (H, W, 3), dtype=np.uint8)
    full = np.tile(np.array([0, 0, W, H], np.uint32), (n, 1))
    one = lambda v: np.full(n, v, np.float32)
    out = {"img": img, "full_roi": full}
    # CropMirrorNormalize 224-style case scaled down: crop 32x24 centre, mean 128 std 1.2, u8 out (unit_tests.cpp:730-735)
    crop = np.stack([orc.fixed_crop(W, H, 32, 24, anchor=(0.5, 0.5)) for _ in range(n)])
    scale, bias = orc.cmn_scale_bias([128, 128, 128], [1.2, 1.2, 1.2], n)
    out["cmn_crop"], out["cmn_scale"], out["cmn_bias"] = crop, scale, bias
    out["cmn_mirror"] = np.array([1, 0], np.uint32)
    out["cmn_u8_nhwc"] = orc.crop_mirror_normalize(img, crop, scale, bias, out["cmn_mirror"], 24, 32, orc.NHWC, orc.UINT8)
    s2, b2 = orc.cmn_scale_bias(wl.MEAN, wl.STD, n)
    out["cmn_scale2"], out["cmn_bias2"] = s2, b2
    out["cmn_f32_nchw"] = orc.crop_mirror_normalize(img, crop, s2, b2, out["cmn_mirror"], 24, 32, orc.NCHW, orc.FP32)
    out["cmn_f16_nchw"] = orc.crop_mirror_normalize(img, crop, s2, b2, out["cmn_mirror"], 24, 32, orc.NCHW, orc.FP16)
    # Resize to 40x30, bilinear and triangular (unit_tests.cpp:605-624 use 400x400)
    dw, dh = np.full(n, 40, np.uint32), np.full(n, 30, np.uint32)
    out["rs_dw"], out["rs_dh"] = dw, dh
    out["resize_bilinear"] = orc.resize(img, full, dw, dh, 30, 40, interp=orc.LINEAR)
    out["resize_triangular"] = orc.resize(img, full, dw, dh, 30, 40, interp=orc.TRIANGULAR)
    out["resize_nearest"] = orc.resize(img, full, dw, dh, 30, 40, interp=orc.NEAREST)
    out["rrc_cmn_f16"] = orc.resize(img, crop, dw, dh, 30, 40, interp=orc.LINEAR, mirror=out["cmn_mirror"], scale=s2, bias=b2,
                                    layout=orc.NCHW, dtype=orc.FP16, flags=orc.F_QUANTIZE_U8)
    # colour family, fixed parameters of unit_tests.cpp:755,763,812,816,820
    out["brightness"] = orc.brightness(img, full, one(1.9), one(20.0))
    out["contrast"] = orc.contrast(img, full, one(30.0), one(80.0))
    out["hue"] = orc.color_twist(img, full, one(1), one(0), one(150.0), one(1))
    out["saturation"] = orc.color_twist(img, full, one(1), one(0), one(0), one(0.3))
    out["color_twist"] = orc.color_twist(img, full, one(0.2), one(10.0), one(100.0), one(0.25))
    # rotate 45 degrees (unit_tests.cpp:751) and warp affine (1,1,.5,.5,7,7) (unit_tests.cpp:772: x0,x1,y0,y1,o0,o1)
    m = np.stack([orc.rotate_matrix(45.0)] * n)
    sw, sh = np.full(n, W, np.uint32), np.full(n, H, np.uint32)
    out["rotate45"] = orc.warp_affine(img, full, m, sw, sh, H, W)
    x0, x1, y0, y1, o0, o1 = 1, 1, .5, .5, 7, 7
    rocal = np.tile(np.array([x0, y0, x1, y1, o0, o1], np.float32), (n, 1))  # rocAL's fill order
    out["warp_rocal_params"] = rocal
    out["warp_affine"] = orc.warp_affine(img, full, np.stack([orc.affine_from_rocal(a) for a in rocal]), sw, sh, H, W)
    # gamma 0.5, exposure 1, colour temperature 70, blend of the image with its 45-degree rotation at 0.5
    # (unit_tests.cpp:759,804,796,767-768)
    out["gamma"] = orc.gamma(img, full, one(0.5))
    out["exposure"] = orc.exposure(img, full, one(1.0))
    out["color_temperature"] = orc.color_temperature(img, full, np.full(n, 70, np.int32))
    out["blend_with_rotate45"] = orc.blend(img, out["rotate45"], full, one(0.5))
    return out


if __name__ == "__main__":
    path = os.path.join(HERE, "augment_golden.npz")
    np.savez_compressed(path, **cases())
    print("wrote", path, os.path.getsize(path), "bytes")
