"""GPU parity of the streaming neighbours of the colour family (Gamma, Exposure, ColorTemperature, Blend) through the
C ABI against the CPU oracle: integer and byte outputs bit-exact, float outputs bit-identical as well (each value is one
fp32 operation or a table entry). Shapes cover the aligned kernels, the general ones (odd widths, windows off the
origin) and the full size of the ColorTwist configuration."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops
from rocal_amd._lib import RmxError

pytestmark = pytest.mark.gpu

COMBOS = [(ops.NHWC, ops.UINT8), (ops.NCHW, ops.UINT8), (ops.NCHW, ops.FP16), (ops.NHWC, ops.FP32), (ops.NHWC, ops.FP16), (ops.NCHW, ops.FP32)]


def _gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _batch(seed, n, h, w, aligned):
    rng = np.random.default_rng(seed)
    img = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    img2 = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    if aligned:
        roi = np.tile(np.array([0, 0, w, h], np.uint32), (n, 1))
        roi[1:, 3] = rng.integers(1, h + 1, n - 1)  # ragged heights, whole 8-pixel groups
        roi[1:, 2] = 8 * rng.integers(1, w // 8 + 1, n - 1)
    else:
        x = rng.integers(0, w // 2, n)
        y = rng.integers(0, h // 2, n)
        roi = np.stack([x, y, rng.integers(1, w - x + 1), rng.integers(1, h - y + 1)], -1).astype(np.uint32)
        roi[0] = (w - 1, h - 1, 1, 1)  # a single pixel that ends on the last byte of its image
    return img, img2, roi


def _run(ctx, cls, n, h, w, layout, dtype, upd, srcs):
    op = cls(ctx, ops.desc(n, h, w, ops.NHWC, ops.UINT8), ops.desc(n, h, w, layout, dtype))
    upd(op)
    out = op.alloc_output()
    op.launch(*[_gpu(s) for s in srcs], out)
    ctx.sync()
    return out.cpu().numpy(), op


def _same(got, exp, what):
    assert got.shape == exp.shape and got.dtype == exp.dtype, (what, got.shape, exp.shape, got.dtype, exp.dtype)
    bad = int((got != exp).sum())
    assert bad == 0, "%s: %d of %d values differ" % (what, bad, got.size)


@pytest.mark.parametrize("aligned", [True, False])
@pytest.mark.parametrize("layout,dtype", COMBOS)
def test_gamma_exposure_temperature_blend(ctx, layout, dtype, aligned):
    n, h, w = 6, 37, 96 if aligned else 101
    img, img2, roi = _batch(7 + int(aligned), n, h, w, aligned)
    rng = np.random.default_rng(99)
    gamma = rng.uniform(0.3, 7.0, n).astype(np.float32)
    factor = rng.uniform(-1.0, 1.5, n).astype(np.float32)
    adj = rng.integers(-99, 100, n).astype(np.int32)
    ratio = rng.uniform(0.0, 1.0, n).astype(np.float32)
    kw = dict(layout=layout, dtype=dtype)
    got, op = _run(ctx, ops.Gamma, n, h, w, layout, dtype, lambda o: o.update(roi, gamma), [img])
    assert op.kernel_name == "rmx_point_kernel"
    _same(got, orc.gamma(img, roi, gamma, **kw), "gamma")
    got, _ = _run(ctx, ops.Exposure, n, h, w, layout, dtype, lambda o: o.update(roi, factor), [img])
    _same(got, orc.exposure(img, roi, factor, **kw), "exposure")
    got, _ = _run(ctx, ops.ColorTemperature, n, h, w, layout, dtype, lambda o: o.update(roi, adj), [img])
    _same(got, orc.color_temperature(img, roi, adj, **kw), "colour temperature")
    got, _ = _run(ctx, ops.Blend, n, h, w, layout, dtype, lambda o: o.update(roi, ratio), [img, img2])
    _same(got, orc.blend(img, img2, roi, ratio, **kw), "blend")


@pytest.mark.parametrize("aligned", [True, False])
@pytest.mark.parametrize("layout,dtype", COMBOS[2:])
def test_colour_family_float_outputs(ctx, layout, dtype, aligned):
    """Brightness, Contrast and ColorTwist writing fp16 / fp32 tensors in both layouts (the coalescing stores of the aligned kernels)."""
    n, h, w = 5, 29, 104 if aligned else 99
    img, _, roi = _batch(21 + int(aligned), n, h, w, aligned)
    rng = np.random.default_rng(5)
    f = lambda lo, hi: rng.uniform(lo, hi, n).astype(np.float32)
    kw = dict(layout=layout, dtype=dtype)
    p = (f(0.3, 2.0), f(-40, 40))
    got, _ = _run(ctx, ops.Brightness, n, h, w, layout, dtype, lambda o: o.update(roi, *p), [img])
    _same(got, orc.brightness(img, roi, *p, **kw), "brightness")
    p = (f(0.3, 2.5), f(0, 255))
    got, _ = _run(ctx, ops.Contrast, n, h, w, layout, dtype, lambda o: o.update(roi, *p), [img])
    _same(got, orc.contrast(img, roi, *p, **kw), "contrast")
    p = (f(0.5, 1.8), f(-30, 30), f(-180, 180), f(0.0, 2.0))
    got, _ = _run(ctx, ops.ColorTwist, n, h, w, layout, dtype, lambda o: o.update(roi, *p), [img])
    _same(got, orc.color_twist(img, roi, *p, **kw), "colour twist")


def test_full_size_u8_batches(ctx):
    """The ColorTwist configuration's shape (256 x 224 x 224 u8 NHWC), every value compared."""
    n, h, w = 256, 224, 224
    rng = np.random.default_rng(2024)
    img = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    img2 = img[::-1].copy()
    roi = np.tile(np.array([0, 0, w, h], np.uint32), (n, 1))
    gamma = rng.uniform(0.3, 7.0, n).astype(np.float32)
    got, op = _run(ctx, ops.Gamma, n, h, w, ops.NHWC, ops.UINT8, lambda o: o.update(roi, gamma), [img])
    _same(got, orc.gamma(img, roi, gamma), "gamma")
    assert op.algorithmic_bytes == 2 * img.size
    ratio = rng.uniform(0.1, 0.9, n).astype(np.float32)
    got, op = _run(ctx, ops.Blend, n, h, w, ops.NHWC, ops.UINT8, lambda o: o.update(roi, ratio), [img, img2])
    _same(got, orc.blend(img, img2, roi, ratio), "blend")
    assert op.algorithmic_bytes == 3 * img.size
    factor = rng.uniform(0.15, 0.95, n).astype(np.float32)
    got, _ = _run(ctx, ops.Exposure, n, h, w, ops.NHWC, ops.UINT8, lambda o: o.update(roi, factor), [img])
    _same(got, orc.exposure(img, roi, factor), "exposure")
    adj = rng.integers(-99, 100, n).astype(np.int32)
    got, _ = _run(ctx, ops.ColorTemperature, n, h, w, ops.NHWC, ops.UINT8, lambda o: o.update(roi, adj), [img])
    _same(got, orc.color_temperature(img, roi, adj), "colour temperature")


def test_gamma_tables_follow_every_update(ctx):
    """The table ring: five updates in a row, each launch reads the table of its own update."""
    n, h, w = 3, 16, 32
    img, _, roi = _batch(5, n, h, w, True)
    sd = ops.desc(n, h, w, ops.NHWC, ops.UINT8)
    op = ops.Gamma(ctx, sd, sd)
    src = _gpu(img)
    outs, gammas = [], []
    for k in range(5):
        g = np.full(n, 0.4 + 0.7 * k, np.float32)
        op.update(roi, g)
        o = op.alloc_output()
        op.launch(src, o)
        outs.append(o)
        gammas.append(g)
    ctx.sync()
    for o, g in zip(outs, gammas):
        _same(o.cpu().numpy(), orc.gamma(img, roi, g), "gamma %g" % g[0])


def test_two_source_protocol_errors(ctx):
    n, h, w = 2, 8, 16
    img, img2, roi = _batch(1, n, h, w, True)
    sd = ops.desc(n, h, w, ops.NHWC, ops.UINT8)
    blend = ops.Blend(ctx, sd, sd)
    blend.update(roi, np.full(n, 0.5, np.float32))
    out = blend.alloc_output()
    with pytest.raises(RmxError, match="two sources"):
        ops.Op.launch(blend, _gpu(img), out)
    with pytest.raises(RmxError, match="ragged"):
        blend.set_ragged_source(np.zeros(n, np.uint64), np.full(n, w, np.uint32), np.full(n, h, np.uint32), img.size)
    bright = ops.Brightness(ctx, sd, sd)
    bright.update(roi, np.ones(n, np.float32), np.zeros(n, np.float32))
    with pytest.raises(RmxError, match="Blend"):
        ops.Blend.launch(bright, _gpu(img), _gpu(img2), out)
    with pytest.raises(RmxError, match="not a Gamma"):
        bright._update("rmx_update_gamma", (roi, np.uint32), (np.ones(n, np.float32), np.float32))
    ctx.sync()


@pytest.mark.parametrize("layout,dtype", [(ops.NCHW, ops.FP32), (ops.NHWC, ops.FP32), (ops.NHWC, ops.FP16), (ops.NHWC, ops.UINT8)])
def test_wide_rows_take_several_tiles(ctx, layout, dtype):
    """Rows wider than one wavefront tile (512 columns): the second tile is narrower than the first and its lanes exchange
    their runs in groups of another size. CropMirrorNormalize with mirrors, Brightness and Gamma on 1160 / 648 columns."""
    n, h, w = 3, 9, 1160
    rng = np.random.default_rng(77)
    img = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    crop = np.array([[0, 0, 1160, 9], [8, 1, 648, 7], [3, 0, 1096, 9]], np.uint32)
    mirror = np.array([1, 0, 1], np.uint32)
    scale = rng.uniform(0.005, 0.03, n * 3).astype(np.float32)
    bias = rng.uniform(-2.5, 0.5, n * 3).astype(np.float32)
    if dtype == ops.UINT8:
        scale[:], bias[:] = 1.0, 0.0
    op = ops.CropMirrorNormalize(ctx, ops.desc(n, h, w, ops.NHWC, ops.UINT8), ops.desc(n, h, w, layout, dtype))
    op.update(crop, scale, bias, mirror)
    out = op.alloc_output()
    op.launch(_gpu(img), out)
    ctx.sync()
    _same(out.cpu().numpy(), orc.crop_mirror_normalize(img, crop, scale, bias, mirror, h, w, layout, dtype), "cmn")
    a, b = rng.uniform(0.3, 2.0, n).astype(np.float32), rng.uniform(-40, 40, n).astype(np.float32)
    got, _ = _run(ctx, ops.Brightness, n, h, w, layout, dtype, lambda o: o.update(crop, a, b), [img])
    _same(got, orc.brightness(img, crop, a, b, layout=layout, dtype=dtype), "brightness")
    g = rng.uniform(0.3, 7.0, n).astype(np.float32)
    got, _ = _run(ctx, ops.Gamma, n, h, w, layout, dtype, lambda o: o.update(crop, g), [img])
    _same(got, orc.gamma(img, crop, g, layout=layout, dtype=dtype), "gamma")


@pytest.mark.parametrize("layout,dtype", COMBOS)
def test_whole_frames_run_as_rows_of_512_pixels(ctx, layout, dtype):
    """Batches in which every sample is a whole frame (64 x 96 = 12 rows of 512 pixels) are handed to the streaming kernels as
    such rows: the colour family, Gamma, Blend, ColorTemperature, CropMirrorNormalize without a mirror and ToTensor, in every
    output format, against the oracle; a mirrored sample keeps CropMirrorNormalize on the image's own rows."""
    n, h, w = 5, 64, 96
    rng = np.random.default_rng(1234 + 10 * layout + dtype)
    img = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    img2 = rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)
    roi = np.tile(np.array([0, 0, w, h], np.uint32), (n, 1))
    f = lambda lo, hi: rng.uniform(lo, hi, n).astype(np.float32)
    gamma, factor, adj, ratio = f(0.3, 3.0), f(-1.0, 1.5), rng.integers(-60, 61, n).astype(np.int32), f(0.0, 1.0)
    alpha, beta, hue, sat = f(0.6, 1.4), f(-20, 20), f(-180, 180), f(0.2, 1.8)
    kw = dict(layout=layout, dtype=dtype)
    cases = [
        (ops.Gamma, lambda op: op.update(roi, gamma), (img,), orc.gamma(img, roi, gamma, **kw)),
        (ops.Blend, lambda op: op.update(roi, ratio), (img, img2), orc.blend(img, img2, roi, ratio, **kw)),
        (ops.Exposure, lambda op: op.update(roi, factor), (img,), orc.exposure(img, roi, factor, **kw)),
        (ops.ColorTemperature, lambda op: op.update(roi, adj), (img,), orc.color_temperature(img, roi, adj, **kw)),
        (ops.Brightness, lambda op: op.update(roi, alpha, beta), (img,), orc.brightness(img, roi, alpha, beta, **kw)),
        (ops.ColorTwist, lambda op: op.update(roi, alpha, beta, hue, sat), (img,), orc.color_twist(img, roi, alpha, beta, hue, sat, **kw)),
    ]
    for cls, upd, srcs, exp in cases:
        got, op = _run(ctx, cls, n, h, w, layout, dtype, upd, srcs)
        assert "flat_rows=12" in op.plan, (cls.__name__, op.plan)
        _same(got, exp, "%s as rows of 512 pixels" % cls.__name__)
    # CropMirrorNormalize of whole frames: as rows of 512 pixels without a mirror, on the image's rows with one
    scale = rng.uniform(0.01, 0.03, (n, 3)).astype(np.float32)
    bias = rng.uniform(-1.0, 1.0, (n, 3)).astype(np.float32)
    if dtype == ops.UINT8:
        scale, bias = np.ones((n, 3), np.float32), rng.integers(-20, 20, (n, 3)).astype(np.float32)
    for mirror in (np.zeros(n, np.uint32), np.array([0, 1, 0, 0, 1], np.uint32)):
        got, op = _run(ctx, ops.CropMirrorNormalize, n, h, w, layout, dtype, lambda op: op.update(roi, scale, bias, mirror), (img,))
        assert ("flat_rows=12" in op.plan) == (not mirror.any()), op.plan
        _same(got, orc.crop_mirror_normalize(img, roi, scale, bias, mirror, h, w, layout, dtype), "CropMirrorNormalize mirror=%s" % mirror.tolist())
    if dtype != ops.UINT8:
        mul, add = np.array([0.5, 0.25, 2.0], np.float32), np.array([-3.0, 7.5, 0.125], np.float32)
        for rev in (False, True):
            op = ops.ToTensor(ctx, ops.desc(n, h, w, ops.NHWC, ops.UINT8), ops.desc(n, h, w, layout, dtype))
            op.update(mul, add, rev)
            assert "flat_rows=12" in op.plan, op.plan
            out = op.alloc_output()
            op.launch(_gpu(img), out)
            ctx.sync()
            _same(out.cpu().numpy(), orc.to_tensor(img, mul, add, rev, layout, dtype), "ToTensor reverse=%s" % rev)
