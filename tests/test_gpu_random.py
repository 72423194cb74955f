"""Seeded random sweeps over shapes and parameters of every kernel family, each case compared bit for bit
with the oracle. Small tensors, many combinations: ragged windows, 1-pixel sizes, up- and down-scaling on both
axes, every layout x dtype, mirrors, fused crops, arbitrary affine maps."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops, workloads as wl

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def _rand_roi(rng, n, H, W, min_w=1, min_h=1):
    roi = np.empty((n, 4), np.uint32)
    for i in range(n):
        w = int(rng.integers(min_w, W + 1))
        h = int(rng.integers(min_h, H + 1))
        roi[i] = (int(rng.integers(0, W - w + 1)), int(rng.integers(0, H - h + 1)), w, h)
    return roi


def _src(rng, n, H, W):
    import torch
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    # an exact-size allocation: nothing behind the last pixel belongs to the tensor
    return img, torch.from_numpy(img.reshape(-1).copy()).cuda().view(n, H, W, 3)


@pytest.mark.parametrize("seed", range(36))
def test_random_resize(ctx, seed):
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(8, 150)), int(rng.integers(8, 200))
    img, src = _src(rng, n, H, W)
    interp = [ops.LINEAR, ops.NEAREST, ops.TRIANGULAR][seed % 3]
    layout = [ops.NCHW, ops.NHWC][int(rng.integers(0, 2))]
    dtype = [ops.UINT8, ops.FP16, ops.FP32][int(rng.integers(0, 3))]
    roi = _rand_roi(rng, n, H, W)
    if rng.random() < 0.5:  # widths that are multiples of 8 reach the aligned fast paths
        dw = (rng.integers(1, 20, n) * 8).astype(np.uint32)
    else:
        dw = rng.integers(1, 160, n).astype(np.uint32)
    dh = rng.integers(1, 120, n).astype(np.uint32)
    if interp == ops.TRIANGULAR and rng.random() < 0.6:  # mostly shrinking: the antialiasing case
        dw = np.maximum(1, np.minimum(dw, roi[:, 2] // rng.integers(1, 4, n))).astype(np.uint32)
        dh = np.maximum(1, np.minimum(dh, roi[:, 3] // rng.integers(1, 4, n))).astype(np.uint32)
    oh, ow = int(dh.max()), int(-(-int(dw.max()) // 8) * 8 if rng.random() < 0.5 else dw.max())
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    norm = dtype != ops.UINT8 and rng.random() < 0.7
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, layout, dtype), interp)
    if norm:
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        exp = orc.resize(img, roi, dw, dh, oh, ow, interp=interp, mirror=mirror, scale=scale, bias=bias, layout=layout, dtype=dtype)
    else:
        op.update(roi, dw, dh, mirror)
        exp = orc.resize(img, roi, dw, dh, oh, ow, interp=interp, mirror=mirror, layout=layout, dtype=dtype)
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(_bits(got), _bits(exp)), "seed %d (%s, %s): %d values differ" % (seed, op.kernel_name, op.plan, int((got != exp).sum()))


@pytest.mark.parametrize("seed", range(16))
def test_random_resize_then_crop_mirror_normalize_fused(ctx, seed):
    """resize (u8) -> CropMirrorNormalize as one launch: the oracle runs the two reference nodes one after the other."""
    rng = np.random.default_rng(2000 + seed)
    n = int(rng.integers(1, 4))
    H, W = int(rng.integers(16, 150)), int(rng.integers(16, 200))
    img, src = _src(rng, n, H, W)
    roi = _rand_roi(rng, n, H, W, 4, 4)
    rw = (rng.integers(2, 20, n) * 8).astype(np.uint32)  # resized size
    rh = rng.integers(8, 120, n).astype(np.uint32)
    crop = np.empty((n, 4), np.uint32)
    for i in range(n):
        cw = int(rng.integers(1, rw[i] // 8 + 1)) * 8
        ch = int(rng.integers(1, rh[i] + 1))
        crop[i] = (int(rng.integers(0, (rw[i] - cw) // 8 + 1)) * 8 if seed % 2 else int(rng.integers(0, rw[i] - cw + 1)), int(rng.integers(0, rh[i] - ch + 1)), cw, ch)
    oh, ow = int(crop[:, 3].max()), int(crop[:, 2].max())
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    layout = [ops.NCHW, ops.NHWC][seed % 2]
    dtype = [ops.FP16, ops.FP32][(seed // 2) % 2]
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, layout, dtype), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
    op.update_cmn(roi, rw, rh, scale, bias, mirror, crop)
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    mid = orc.resize(img, roi, rw, rh, int(rh.max()), int(rw.max()), interp=orc.LINEAR)
    exp = orc.crop_mirror_normalize(mid, crop, scale, bias, mirror, oh, ow, layout, dtype)
    got = out.cpu().numpy()
    assert np.array_equal(_bits(got), _bits(exp)), "seed %d (%s, %s): %d values differ" % (seed, op.kernel_name, op.plan, int((got != exp).sum()))


@pytest.mark.parametrize("seed", range(16))
def test_random_crop_mirror_normalize(ctx, seed):
    rng = np.random.default_rng(3000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(4, 120)), int(rng.integers(4, 200))
    img, src = _src(rng, n, H, W)
    crop = _rand_roi(rng, n, H, W)
    if seed % 2:
        crop[:, 2] = np.maximum(8, crop[:, 2] // 8 * 8)
        crop[:, 0] = np.minimum(crop[:, 0], max(W, 8) - crop[:, 2]) if W >= 8 else 0
    if W < 8 or (crop[:, 0] + crop[:, 2] > W).any():
        crop = _rand_roi(rng, n, H, W)
    oh, ow = int(crop[:, 3].max()), int(crop[:, 2].max())
    layout = [ops.NCHW, ops.NHWC][int(rng.integers(0, 2))]
    dtype = [ops.UINT8, ops.FP16, ops.FP32][seed % 3]
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    scale = rng.uniform(0.005, 0.03, n * 3).astype(np.float32)
    bias = rng.uniform(-2.5, 0.5, n * 3).astype(np.float32)
    if dtype == ops.UINT8:
        scale[:] = 1.0
        bias[:] = 0.0
    op = ops.CropMirrorNormalize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, layout, dtype))
    op.update(crop, scale, bias, mirror)
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    exp = orc.crop_mirror_normalize(img, crop, scale, bias, mirror, oh, ow, layout, dtype)
    got = out.cpu().numpy()
    assert np.array_equal(_bits(got), _bits(exp)), "seed %d (%s): %d values differ" % (seed, op.plan, int((got != exp).sum()))


@pytest.mark.parametrize("seed", range(20))
def test_random_colour(ctx, seed):
    rng = np.random.default_rng(4000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(4, 100)), int(rng.integers(4, 160))
    img, src = _src(rng, n, H, W)
    if seed % 4 == 0:  # greys and saturated primaries among the pixels
        img[:, ::3] = img[:, ::3, :, :1]
        img[:, 1::5, ::2] = (255, 0, 0)
        import torch
        src = torch.from_numpy(img.reshape(-1).copy()).cuda().view(n, H, W, 3)
    roi = _rand_roi(rng, n, H, W)
    if seed % 2:
        roi[:, 2] = np.maximum(8, roi[:, 2] // 8 * 8)
        if W < 8 or (roi[:, 0] + roi[:, 2] > W).any():
            roi[:, 0] = 0
            roi[:, 2] = max(1, W // 8 * 8) if W >= 8 else W
    f = lambda lo, hi: rng.uniform(lo, hi, n).astype(np.float32)
    kind = seed % 5
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)
    if kind == 0:
        p = (f(0.5, 1.8), f(-30, 30), f(-180, 180), f(0.0, 2.0))
        op, exp = ops.ColorTwist(ctx, sd, sd), orc.color_twist(img, roi, *p)
    elif kind == 1:
        p = (f(0.3, 2.0), f(-40, 40))
        op, exp = ops.Brightness(ctx, sd, sd), orc.brightness(img, roi, *p)
    elif kind == 2:
        p = (f(0.3, 2.5), f(0, 255))
        op, exp = ops.Contrast(ctx, sd, sd), orc.contrast(img, roi, *p)
    elif kind == 3:
        p = (f(-360, 360),)
        one, zero = np.ones(n, np.float32), np.zeros(n, np.float32)
        op, exp = ops.Hue(ctx, sd, sd), orc.color_twist(img, roi, one, zero, p[0], one)
    else:
        p = (f(0.0, 3.0),)
        one, zero = np.ones(n, np.float32), np.zeros(n, np.float32)
        op, exp = ops.Saturation(ctx, sd, sd), orc.color_twist(img, roi, one, zero, zero, p[0])
    op.update(roi, *p)
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(got, exp), "seed %d kind %d (%s): %d values differ" % (seed, kind, op.plan, int((got != exp).sum()))


@pytest.mark.parametrize("w4", [False, True])
@pytest.mark.parametrize("seed", range(24))
def test_random_warp(ctx, seed, w4):
    """w4: a source width that is a multiple of 4 (rows start at one byte phase), which takes the form of the kernel that
    loads the source boxes straight into LDS as packed bytes."""
    rng = np.random.default_rng(5000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(4, 140)), int(rng.integers(4, 180))
    if w4:
        W = (W + 3) // 4 * 4
    img, src = _src(rng, n, H, W)
    roi = _rand_roi(rng, n, H, W)
    dw = np.minimum(rng.integers(1, 200, n), W).astype(np.uint32)
    dh = np.minimum(rng.integers(1, 150, n), H).astype(np.uint32)
    if seed % 3 == 0:
        dw = np.maximum(8, dw // 8 * 8).astype(np.uint32) if W >= 8 else dw
    affine = np.empty((n, 6), np.float32)
    for i in range(n):
        ang = rng.uniform(-np.pi, np.pi)
        sx, sy = rng.uniform(0.2, 4.0, 2) if seed % 4 else rng.uniform(0.8, 1.25, 2)
        c, s = np.cos(ang), np.sin(ang)
        # rocAL's order x0,y0,x1,y1,o0,o1 with M = [[x0,x1,o0],[y0,y1,o1]]
        affine[i] = (c * sx, s * sx, -s * sy, c * sy, rng.uniform(-20, 20), rng.uniform(-20, 20))
    interp = [ops.LINEAR, ops.NEAREST][seed % 2]
    m = np.stack([orc.affine_from_rocal(a) for a in affine])
    exp = orc.warp_affine(img, roi, m, dw, dh, H, W, interp=interp)
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)
    op = ops.WarpAffine(ctx, sd, sd, interp)
    op.update(roi, affine, dw, dh)
    out = op.alloc_output()
    op.launch(src, out)
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(got, exp), "seed %d (%s): %d values differ" % (seed, op.plan, int((got != exp).sum()))


def _ragged(rng, n, H, W):
    """n images of their own sizes (<= H x W): packed one after the other at arbitrary byte offsets of one buffer,
    and the same images in the top-left corners of a padded [n,H,W,3] tensor for the oracle."""
    import torch
    ws = rng.integers(max(1, W // 3), W + 1, n).astype(np.uint32)
    hs = rng.integers(max(1, H // 3), H + 1, n).astype(np.uint32)
    padded = np.zeros((n, H, W, 3), np.uint8)
    chunks, offsets, pos = [], [], int(rng.integers(0, 2)) * 4
    lead = pos
    for i in range(n):
        im = rng.integers(0, 256, (hs[i], ws[i], 3), dtype=np.uint8)
        padded[i, :hs[i], :ws[i]] = im
        gap = int(rng.integers(0, 6))
        offsets.append(pos + gap)
        chunks.append(np.zeros(gap, np.uint8))
        chunks.append(im.reshape(-1))
        pos += gap + im.size
    buf = np.concatenate([np.zeros(lead, np.uint8)] + chunks)
    return padded, torch.from_numpy(buf).cuda(), np.array(offsets, np.uint64), ws, hs, buf.size


def _roi_in(rng, ws, hs):
    roi = np.empty((len(ws), 4), np.uint32)
    for i, (w, h) in enumerate(zip(ws, hs)):
        rw, rh = int(rng.integers(1, w + 1)), int(rng.integers(1, h + 1))
        roi[i] = (int(rng.integers(0, w - rw + 1)), int(rng.integers(0, h - rh + 1)), rw, rh)
    return roi


@pytest.mark.parametrize("seed", range(30))
def test_random_ops_on_a_ragged_source(ctx, seed):
    """Every kernel family reading tightly packed images of different sizes instead of a padded tensor."""
    rng = np.random.default_rng(6000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(12, 140)), int(rng.integers(12, 180))
    padded, buf, offsets, ws, hs, nbytes = _ragged(rng, n, H, W)
    roi = _roi_in(rng, ws, hs)
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)
    family = seed % 5
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    if family in (0, 1, 2):  # resize: linear (also the aligned fast path), nearest, triangular
        interp = [ops.LINEAR, ops.NEAREST, ops.TRIANGULAR][family]
        dw = (rng.integers(1, 16, n) * 8).astype(np.uint32) if seed % 2 else rng.integers(1, 120, n).astype(np.uint32)
        dh = rng.integers(1, 100, n).astype(np.uint32)
        oh, ow = int(dh.max()), int(dw.max())
        op = ops.Resize(ctx, sd, ops.desc(n, oh, ow, ops.NCHW, ops.FP16), interp)
        op.set_ragged_source(offsets, ws, hs, nbytes)
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        exp = orc.resize(padded, roi, dw, dh, oh, ow, interp=interp, mirror=mirror, scale=scale, bias=bias, layout=orc.NCHW, dtype=orc.FP16)
    elif family == 3:
        if seed % 2:
            roi[:, 2] = np.maximum(1, roi[:, 2] // 8 * 8)
        oh, ow = int(roi[:, 3].max()), int(roi[:, 2].max())
        op = ops.CropMirrorNormalize(ctx, sd, ops.desc(n, oh, ow, ops.NCHW, ops.FP32))
        op.set_ragged_source(offsets, ws, hs, nbytes)
        op.update(roi, scale, bias, mirror)
        exp = orc.crop_mirror_normalize(padded, roi, scale, bias, mirror, oh, ow, orc.NCHW, orc.FP32)
    else:
        if seed % 2:
            f = lambda lo, hi: rng.uniform(lo, hi, n).astype(np.float32)
            p = (f(0.5, 1.8), f(-30, 30), f(-180, 180), f(0.0, 2.0))
            op = ops.ColorTwist(ctx, sd, sd)
            op.set_ragged_source(offsets, ws, hs, nbytes)
            op.update(roi, *p)
            exp = orc.color_twist(padded, roi, *p)
        else:
            affine = np.empty((n, 6), np.float32)
            for i in range(n):
                ang, sc = rng.uniform(-np.pi, np.pi), rng.uniform(0.5, 2.0)
                affine[i] = (np.cos(ang) * sc, np.sin(ang) * sc, -np.sin(ang) * sc, np.cos(ang) * sc, rng.uniform(-8, 8), rng.uniform(-8, 8))
            dw = np.minimum(rng.integers(1, 160, n), W).astype(np.uint32)
            dh = np.minimum(rng.integers(1, 120, n), H).astype(np.uint32)
            op = ops.WarpAffine(ctx, sd, sd, ops.LINEAR)
            op.set_ragged_source(offsets, ws, hs, nbytes)
            op.update(roi, affine, dw, dh)
            exp = orc.warp_affine(padded, roi, np.stack([orc.affine_from_rocal(a) for a in affine]), dw, dh, H, W, interp=orc.LINEAR)
    out = op.alloc_output()
    op.launch(buf, out)
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(_bits(got), _bits(exp)), "seed %d family %d (%s, %s): %d values differ" % (seed, family, op.kernel_name, op.plan, int((got != exp).sum()))
    # and back to the padded tensor with the same op
    import torch
    op.set_ragged_source(None, None, None, 0)
    if family in (0, 1, 2):
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
    elif family == 3:
        op.update(roi, scale, bias, mirror)
    elif seed % 2:
        op.update(roi, *p)
    else:
        op.update(roi, affine, dw, dh)
    out2 = op.alloc_output()
    op.launch(torch.from_numpy(padded).cuda(), out2)
    ctx.sync()
    assert np.array_equal(_bits(out2.cpu().numpy()), _bits(exp))


@pytest.mark.parametrize("seed", range(24))
def test_random_gamma_exposure_temperature_blend(ctx, seed):
    """The streaming neighbours of the colour family on exact-size buffers; every third case reads a ragged source
    (the one-input ops) or, for Blend, windows that end on the last byte of both batches."""
    import torch
    rng = np.random.default_rng(7000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(4, 100)), int(rng.integers(4, 160))
    kind = seed % 4
    ragged = seed % 3 == 0 and kind != 3
    layout = [ops.NHWC, ops.NCHW][int(rng.integers(0, 2))]
    dtype = [ops.UINT8, ops.UINT8, ops.FP16, ops.FP32][int(rng.integers(0, 4))]
    if ragged:
        img, src, offsets, ws, hs, nbytes = _ragged(rng, n, H, W)
        roi = _roi_in(rng, ws, hs)
    else:
        img, src = _src(rng, n, H, W)
        roi = _rand_roi(rng, n, H, W)
        if seed % 2 and W >= 8:  # whole 8-pixel groups reach the aligned kernels
            roi[:, 2] = np.maximum(8, roi[:, 2] // 8 * 8)
            roi[:, 0] = np.minimum(roi[:, 0], W - roi[:, 2])
    if kind == 3:
        roi[0] = (W - roi[0, 2], H - roi[0, 3], roi[0, 2], roi[0, 3])  # ends on the last pixel of the first image
        roi[-1] = (W - 1, H - 1, 1, 1)
    oh, ow = H, (W + 7) // 8 * 8 if seed % 2 else W
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, layout, dtype)
    f = lambda lo, hi: rng.uniform(lo, hi, n).astype(np.float32)
    kw = dict(layout=layout, dtype=dtype)

    def fit(exp):  # the oracle writes an H x W destination; the op's may be wider
        full = np.zeros((n, 3, oh, ow) if layout == ops.NCHW else (n, oh, ow, 3), exp.dtype)
        if layout == ops.NCHW:
            full[:, :, :H, :W] = exp
        else:
            full[:, :H, :W] = exp
        return full

    srcs = [src]
    if kind == 0:
        p = f(0.3, 7.0)
        op, exp = ops.Gamma(ctx, sd, dd), orc.gamma(img, roi, p, **kw)
    elif kind == 1:
        p = f(-2.0, 2.0)
        op, exp = ops.Exposure(ctx, sd, dd), orc.exposure(img, roi, p, **kw)
    elif kind == 2:
        p = rng.integers(-99, 100, n).astype(np.int32)
        op, exp = ops.ColorTemperature(ctx, sd, dd), orc.color_temperature(img, roi, p, **kw)
    else:
        p = f(0.0, 1.0)
        img2, src2 = _src(rng, n, H, W)
        srcs.append(src2)
        op, exp = ops.Blend(ctx, sd, dd), orc.blend(img, img2, roi, p, **kw)
    if ragged:
        op.set_ragged_source(offsets, ws, hs, nbytes)
    op.update(roi, p)
    out = op.alloc_output()
    op.launch(*srcs, out)
    ctx.sync()
    got = out.cpu().numpy()
    exp = fit(exp)
    assert np.array_equal(_bits(got), _bits(exp)), "seed %d kind %d (%s, %s): %d values differ" % (seed, kind, op.kernel_name, op.plan, int((got != exp).sum()))
