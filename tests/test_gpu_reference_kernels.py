"""Pins the oracle's resize and to_tensor restatements against the reference's OWN in-tree HIP
kernels (rocAL/rocAL_hip/rocal_hip_kernels.cpp), compiled from the reference tree into
oracle/_ref/librocal_hip_ref.so by oracle/Makefile, and checks the HIP path against the committed
golden vectors without the oracle. The reference kernels are the only executable arithmetic for
this path inside the reference tree; RPP itself is not available."""
import ctypes as C
import os

import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.path.join(ROOT, "oracle", "_ref", "librocal_hip_ref.so")


@pytest.fixture(scope="module")
def ref():
    if not os.path.exists(REF):
        pytest.skip("oracle/_ref was not built (the reference tree was absent at build time)")
    import torch  # noqa: F401  (its bundled HIP runtime must be the one the reference library binds to)
    lib = C.CDLL(REF)
    lib.ref_resize_tensor.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_void_p, C.c_void_p, C.c_uint, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t]
    lib.ref_copy_int8_to_tensor.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_uint, C.c_uint, C.c_uint, C.c_uint,
                                            C.c_void_p, C.c_void_p, C.c_uint, C.c_uint]
    return lib


def _dev_i64(a):
    import torch
    return torch.tensor(np.asarray(a, np.int64), device="cuda")


def _run_ref_resize(ref, img, sw, sh, dw, dh, max_dw, max_dh):
    """img: [n, H, W, c] u8 (c = 3 packed or 1 planar). Returns [n, max_dh, max_dw, c]."""
    import torch
    n, H, W, c = img.shape
    src = torch.zeros(img.size + 64, dtype=torch.uint8, device="cuda")
    src[:img.size] = torch.from_numpy(img.reshape(-1)).cuda()
    dst = torch.zeros(n * max_dh * max_dw * c + 64, dtype=torch.uint8, device="cuda")
    args = [_dev_i64(sw), _dev_i64(sh), _dev_i64(dw), _dev_i64(dh), _dev_i64([W * c] * n), _dev_i64([i * H * W * c for i in range(n)])]
    torch.cuda.synchronize()
    rc = ref.ref_resize_tensor(None, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), n, *[C.c_void_p(a.data_ptr()) for a in args],
                               c, W, H, max_dw, max_dh)
    ref.ref_error_name.restype = C.c_char_p
    assert rc == 0, ref.ref_error_name(rc)
    return dst[:n * max_dh * max_dw * c].cpu().numpy().reshape(n, max_dh, max_dw, c)


def test_oracle_bilinear_matches_reference_hip_kernel(ref):
    """rocal_hip_kernels.cpp:311-332,447-485 (resize_bilinear_pkd_hip_tensor).

    The reference kernel writes `(float4)scalar` and `(float2)1.0f` expecting a broadcast. The HIP
    headers of this toolchain build such a cast as (scalar, 0, 0, 0), so in a build made here only
    lane 0 of every 8-pixel group gets its source x, and the "next row" of the 2x2 footprint is the
    same row again. What is still the reference's arithmetic, and what this test pins, is therefore:
    the x source-coordinate law `d*ratio + (ratio-1)/2 + lo`, the horizontal weights and the fmaf
    chain, the clamp of both neighbours to hi-1 (oracle flag F_BILINEAR_EDGE_QUIRK) and the
    round-to-nearest-even u8 store - on destination columns that are multiples of 8, with a
    vertical ratio of exactly 1 so that the bottom row carries weight 0. The y law is the same
    code with the axes swapped and is pinned by the closed forms in test_oracle_cpu.py."""
    rng = np.random.default_rng(31)
    n, H, W = 3, 97, 131
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    sw, sh = [131, 100, 77], [97, 80, 64]
    dw, dh = [64, 160, 40], list(sh)
    got = _run_ref_resize(ref, img, sw, sh, dw, dh, 160, 97)
    roi = np.array([[0, 0, sw[i], sh[i]] for i in range(n)], np.uint32)
    exp = orc.resize(img, roi, dw, dh, 97, 160, interp=orc.LINEAR, flags=orc.F_BILINEAR_EDGE_QUIRK)
    for i in range(n):
        g, e = (a[i, :dh[i], :dw[i]:8].astype(np.int32) for a in (got, exp))
        # the quirk clamps the row to hi-1 as well: the last row reads row hi-1 in both
        d = np.abs(g - e)
        assert d.max() == 0, "sample %d differs by %d at %s" % (i, d.max(), np.argwhere(d > 0)[:4].tolist())
    # upscaling sample (ratio < 1) exercises the low clamp, downscaling ones the interior
    assert dw[1] > sw[1] and dw[0] < sw[0]


def test_oracle_triangular_matches_reference_hip_kernel(ref):
    """rocal_hip_kernels.cpp:515-589 (resize_generic_pln1_hip_tensor): single channel, 2-D loop,
    truncating store -> oracle flags F_TRI_2D | F_ROUND_TRUNC."""
    rng = np.random.default_rng(32)
    n, H, W = 2, 120, 150
    img = rng.integers(0, 256, (n, H, W, 1), dtype=np.uint8)
    sw, sh = [150, 90], [120, 100]
    dw, dh = [50, 64], [40, 24]
    got = _run_ref_resize(ref, img, sw, sh, dw, dh, 64, 40)
    roi = np.array([[0, 0, sw[i], sh[i]] for i in range(n)], np.uint32)
    exp = orc.resize(img, roi, dw, dh, 40, 64, interp=orc.TRIANGULAR, flags=orc.F_TRI_2D | orc.F_ROUND_TRUNC)
    sep = orc.resize(img, roi, dw, dh, 40, 64, interp=orc.TRIANGULAR)
    for i in range(n):
        g, e, s = (a[i, :dh[i], :dw[i]].astype(np.int32) for a in (got, exp, sep))
        d = np.abs(g - e)
        assert d.max() <= 1 and (d > 0).mean() < 0.05, (d.max(), (d > 0).mean())
        # the oracle's default (separable, round-to-nearest) stays within one grey level of the reference
        assert np.abs(g - s).max() <= 1


@pytest.mark.parametrize("nchw,fp16,reverse", [(1, 0, 0), (1, 1, 0), (1, 0, 1), (0, 0, 0), (1, 1, 1)])
def test_oracle_to_tensor_matches_reference_hip_kernel(ref, nchw, fp16, reverse):
    """rocal_hip_kernels.cpp:40-309 (Hip_CopyInt8ToNCHW/NHWC): out = u8*mul + add, bit-exact."""
    import torch
    rng = np.random.default_rng(33)
    n, H, W = 3, 33, 47
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    mul = np.array([1 / 58.395, 1 / 57.12, 1 / 57.375], np.float32)
    add = np.array([-123.675 / 58.395, -116.28 / 57.12, -103.53 / 57.375], np.float32)
    src = torch.from_numpy(img).cuda()
    dst = torch.zeros(n * 3 * H * W, dtype=torch.float16 if fp16 else torch.float32, device="cuda")
    torch.cuda.synchronize()
    rc = ref.ref_copy_int8_to_tensor(None, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), nchw, n, 3, H, W,
                                     mul.ctypes.data_as(C.c_void_p), add.ctypes.data_as(C.c_void_p), reverse, fp16)
    assert rc == 0
    got = dst.cpu().numpy().reshape((n, 3, H, W) if nchw else (n, H, W, 3))
    exp = orc.to_tensor(img, mul, add, reverse_channels=bool(reverse), layout=orc.NCHW if nchw else orc.NHWC,
                        dtype=orc.FP16 if fp16 else orc.FP32)
    assert np.array_equal(got.view(np.uint16 if fp16 else np.uint32), exp.view(np.uint16 if fp16 else np.uint32))


def test_hip_path_reproduces_golden_vectors(ctx):
    """HIP kernels against tests/golden/augment_golden.npz, without the oracle in the loop."""
    import torch
    g = np.load(os.path.join(ROOT, "tests", "golden", "augment_golden.npz"))
    img = g["img"]
    n, H, W, _ = img.shape
    gi = torch.from_numpy(img).cuda()
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)

    def run(op, *args, method="update"):
        getattr(op, method)(*args)
        out = op.alloc_output()
        op.launch(gi, out)
        ctx.sync()
        return out.cpu().numpy()

    def same(a, b, name):
        assert a.shape == b.shape and np.array_equal(a.view(np.uint8), b.view(np.uint8)), name

    full, crop = g["full_roi"], g["cmn_crop"]
    same(run(ops.CropMirrorNormalize(ctx, sd, ops.desc(n, 24, 32, ops.NHWC, ops.UINT8)), crop, g["cmn_scale"], g["cmn_bias"], g["cmn_mirror"]),
         g["cmn_u8_nhwc"], "cmn u8")
    same(run(ops.CropMirrorNormalize(ctx, sd, ops.desc(n, 24, 32, ops.NCHW, ops.FP32)), crop, g["cmn_scale2"], g["cmn_bias2"], g["cmn_mirror"]),
         g["cmn_f32_nchw"], "cmn f32")
    same(run(ops.CropMirrorNormalize(ctx, sd, ops.desc(n, 24, 32, ops.NCHW, ops.FP16)), crop, g["cmn_scale2"], g["cmn_bias2"], g["cmn_mirror"]),
         g["cmn_f16_nchw"], "cmn f16")
    rd = ops.desc(n, 30, 40, ops.NHWC, ops.UINT8)
    for interp, key in ((ops.LINEAR, "resize_bilinear"), (ops.TRIANGULAR, "resize_triangular"), (ops.NEAREST, "resize_nearest")):
        same(run(ops.Resize(ctx, sd, rd, interp), full, g["rs_dw"], g["rs_dh"]), g[key], key)
    fused = ops.Resize(ctx, sd, ops.desc(n, 30, 40, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
    same(run(fused, crop, g["rs_dw"], g["rs_dh"], g["cmn_scale2"], g["cmn_bias2"], g["cmn_mirror"], method="update_cmn"), g["rrc_cmn_f16"], "rrc+cmn")
    one = lambda v: np.full(n, v, np.float32)
    same(run(ops.Brightness(ctx, sd, sd), full, one(1.9), one(20.0)), g["brightness"], "brightness")
    same(run(ops.Contrast(ctx, sd, sd), full, one(30.0), one(80.0)), g["contrast"], "contrast")
    same(run(ops.Hue(ctx, sd, sd), full, one(150.0)), g["hue"], "hue")
    same(run(ops.Saturation(ctx, sd, sd), full, one(0.3)), g["saturation"], "saturation")
    same(run(ops.ColorTwist(ctx, sd, sd), full, one(0.2), one(10.0), one(100.0), one(0.25)), g["color_twist"], "color twist")
    size = (np.full(n, W, np.uint32), np.full(n, H, np.uint32))
    same(run(ops.Rotate(ctx, sd, sd, ops.LINEAR), full, one(45.0), *size), g["rotate45"], "rotate")
    same(run(ops.WarpAffine(ctx, sd, sd, ops.LINEAR), full, g["warp_rocal_params"], *size), g["warp_affine"], "warp affine")
    same(run(ops.Gamma(ctx, sd, sd), full, one(0.5)), g["gamma"], "gamma")
    same(run(ops.Exposure(ctx, sd, sd), full, one(1.0)), g["exposure"], "exposure")
    same(run(ops.ColorTemperature(ctx, sd, sd), full, np.full(n, 70, np.int32)), g["color_temperature"], "colour temperature")
    blend = ops.Blend(ctx, sd, sd)
    blend.update(full, one(0.5))
    out = blend.alloc_output()
    blend.launch(gi, torch.from_numpy(g["rotate45"]).cuda(), out)
    ctx.sync()
    same(out.cpu().numpy(), g["blend_with_rotate45"], "blend")


@pytest.mark.parametrize("nchw,fp16,reverse", [(1, 0, 0), (1, 1, 1), (0, 0, 0), (0, 0, 1), (1, 1, 0)])
def test_hip_to_tensor_matches_reference_hip_kernel(ctx, ref, nchw, fp16, reverse):
    """The ToTensor op of the library against the reference's own device kernel for the same step
    (rocal_hip_kernels.cpp:40-308), bit for bit, and against the oracle. The interleaved fp16 variant
    of the reference is left out: it addresses destination rows at y*W + 3x (rocal_hip_kernels.cpp:112),
    so its rows overwrite one another; that combination is checked against the oracle below."""
    import torch
    rng = np.random.default_rng(34)
    n, H, W = 4, 40, 56
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    mul = np.array([1 / 58.395, 1 / 57.12, 1 / 57.375], np.float32)
    add = np.array([-123.675 / 58.395, -116.28 / 57.12, -103.53 / 57.375], np.float32)
    src = torch.from_numpy(img).cuda()
    layout, dtype = (ops.NCHW if nchw else ops.NHWC), (ops.FP16 if fp16 else ops.FP32)
    op = ops.ToTensor(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, H, W, layout, dtype))
    op.update(mul, add, reverse_channels=bool(reverse))
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    got = out.cpu().numpy()
    dst = torch.zeros(n * 3 * H * W, dtype=torch.float16 if fp16 else torch.float32, device="cuda")
    torch.cuda.synchronize()
    rc = ref.ref_copy_int8_to_tensor(None, C.c_void_p(src.data_ptr()), C.c_void_p(dst.data_ptr()), nchw, n, 3, H, W,
                                     mul.ctypes.data_as(C.c_void_p), add.ctypes.data_as(C.c_void_p), reverse, fp16)
    assert rc == 0
    theirs = dst.cpu().numpy().reshape(got.shape)
    bits = np.uint16 if fp16 else np.uint32
    assert np.array_equal(got.view(bits), theirs.view(bits))
    exp = orc.to_tensor(img, mul, add, reverse_channels=bool(reverse), layout=orc.NCHW if nchw else orc.NHWC, dtype=orc.FP16 if fp16 else orc.FP32)
    assert np.array_equal(got.view(bits), exp.view(bits))


@pytest.mark.parametrize("reverse", [0, 1])
def test_hip_to_tensor_interleaved_fp16_matches_oracle(ctx, reverse):
    import torch
    rng = np.random.default_rng(35)
    n, H, W = 3, 21, 43   # odd width: the byte-wise loaders, not the aligned variant
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    mul = np.array([1 / 255.0, 0.5, 2.0], np.float32)
    add = np.array([0.0, -1.0, 0.25], np.float32)
    op = ops.ToTensor(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, H, W, ops.NHWC, ops.FP16))
    op.update(mul, add, reverse_channels=bool(reverse))
    out = op.alloc_output()
    op.launch(torch.from_numpy(img).cuda(), out)
    ctx.sync()
    exp = orc.to_tensor(img, mul, add, reverse_channels=bool(reverse), layout=orc.NHWC, dtype=orc.FP16)
    assert np.array_equal(out.cpu().numpy().view(np.uint16), exp.view(np.uint16))
