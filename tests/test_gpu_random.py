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


@pytest.mark.parametrize("seed", range(24))
def test_random_warp(ctx, seed):
    rng = np.random.default_rng(5000 + seed)
    n = int(rng.integers(1, 5))
    H, W = int(rng.integers(4, 140)), int(rng.integers(4, 180))
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
