"""GPU parity of Normalize (statistics computed on the device or given) and Transpose through the C ABI against the oracle, bit
for bit: ragged windows, both axis masks, every destination format of the streaming kernel, constant samples, full size."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops
from rocal_amd._lib import RmxError

pytestmark = pytest.mark.gpu


def _gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _windows(got, exp, roi, layout):
    for i in range(got.shape[0]):
        w, h = int(roi[i, 2]), int(roi[i, 3])
        g = got[i, :, :h, :w] if layout == ops.NCHW else got[i, :h, :w]
        e = exp[i, :, :h, :w] if layout == ops.NCHW else exp[i, :h, :w]
        assert np.array_equal(g.view(np.uint8), e.view(np.uint8)), "sample %d: %d values differ" % (i, int((g != e).sum()))


@pytest.mark.parametrize("layout,dtype", [(ops.NHWC, ops.FP32), (ops.NCHW, ops.FP32), (ops.NHWC, ops.FP16), (ops.NCHW, ops.FP16)])
@pytest.mark.parametrize("mask", [3, 7])
def test_normalize_with_computed_statistics(ctx, layout, dtype, mask):
    rng = np.random.default_rng(100 + mask)
    n, H, W = 7, 61, 88
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    img[3] = 200  # a constant sample: deviation 0
    img[4, :, :, 1] = 9  # one constant channel
    roi = np.array([[0, 0, 88, 61], [5, 7, 40, 33], [0, 0, 88, 1], [0, 0, 16, 16], [8, 0, 80, 61], [87, 60, 1, 1], [1, 2, 77, 50]], np.uint32)
    exp = orc.normalize(img, roi, axis_mask=mask, scale=1.5, shift=0.25, layout=layout, dtype=dtype)
    op = ops.Normalize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, H, W, layout, dtype))
    op.update(roi, axis_mask=mask, scale=1.5, shift=0.25)
    out = op.alloc_output()
    src = _gpu(img)
    for rep in range(2):  # the counters are cleared by every launch
        op.launch(src, out)
        ctx.sync()
        _windows(out.cpu().numpy(), exp, roi, layout)


def test_normalize_with_given_statistics_and_errors(ctx):
    rng = np.random.default_rng(7)
    n, H, W = 4, 40, 48
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.tile(np.array([0, 0, W, H], np.uint32), (n, 1))
    op = ops.Normalize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, H, W, ops.NHWC, ops.FP32))
    src, out = _gpu(img), None
    for kw in (dict(mean=[123.675, 116.28, 103.53], stddev=[58.395, 57.12, 57.375]), dict(mean=[128.0], stddev=[64.0], scale=2.0, shift=-1.0),
               dict(mean=[0.0], axis_mask=7), dict(stddev=[10.0, 20.0, 30.0])):
        exp = orc.normalize(img, roi, layout=ops.NHWC, dtype=ops.FP32, **kw)
        op.update(roi, **kw)
        out = op.alloc_output()
        op.launch(src, out)
        ctx.sync()
        _windows(out.cpu().numpy(), exp, roi, ops.NHWC)
    with pytest.raises(RmxError, match="axis mask"):
        op.update(roi, axis_mask=4)
    with pytest.raises(RmxError, match="is 0"):
        op.update(roi, mean=[1.0], stddev=[0.0])


def test_normalize_full_size_batch(ctx):
    rng = np.random.default_rng(8)
    n = 64
    img = rng.integers(0, 256, (n, 224, 224, 3), dtype=np.uint8)
    roi = np.tile(np.array([0, 0, 224, 224], np.uint32), (n, 1))
    exp = orc.normalize(img, roi, layout=ops.NCHW, dtype=ops.FP16)
    op = ops.Normalize(ctx, ops.desc(n, 224, 224, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16))
    op.update(roi)
    out = op.alloc_output()
    op.launch(_gpu(img), out)
    ctx.sync()
    got = out.cpu().numpy()
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), "%d values differ" % int((got != exp).sum())


@pytest.mark.parametrize("perm", [(0, 1, 2), (2, 0, 1), (1, 0, 2), (2, 1, 0)])
@pytest.mark.parametrize("dtype", [ops.UINT8, ops.FP16, ops.FP32])
def test_transpose_permutations(ctx, perm, dtype):
    """Expected values are numpy's transpose of each sample's window (an integer gather: exact in every destination type)."""
    rng = np.random.default_rng(50)
    n, H, W = 5, 70, 45
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, 45, 70], [3, 5, 33, 40], [0, 0, 1, 70], [10, 60, 35, 10], [44, 69, 1, 1]], np.uint32)
    swap = perm in ((1, 0, 2), (2, 1, 0))
    first = perm[0] == 2
    oh, ow = (W, H) if swap else (H, W)
    layout = ops.NCHW if first else ops.NHWC
    op = ops.Transpose(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, layout, dtype), perm)
    op.update(roi)
    out = op.alloc_output(fill=3)
    op.launch(_gpu(img), out)
    ctx.sync()
    got = out.cpu().numpy()
    np_dt = {ops.UINT8: np.uint8, ops.FP16: np.float16, ops.FP32: np.float32}[dtype]
    for i in range(n):
        x, y, w, h = [int(v) for v in roi[i]]
        win = img[i, y:y + h, x:x + w].transpose(perm).astype(np_dt)
        g = got[i, :, :win.shape[1], :win.shape[2]] if first else got[i, :win.shape[0], :win.shape[1]]
        assert np.array_equal(g, win), "sample %d perm %s" % (i, perm)
    # outside the written windows the destination keeps its fill value
    x, y, w, h = [int(v) for v in roi[1]]
    tail = got[1, :, (w if swap else h):] if first else got[1, (w if swap else h):]
    assert (tail == 3).all()


def test_transpose_refuses_what_the_node_refuses(ctx):
    sd = ops.desc(2, 8, 8, ops.NHWC, ops.UINT8)
    with pytest.raises(RmxError, match="channel axis"):
        ops.Transpose(ctx, sd, ops.desc(2, 8, 8, ops.NHWC, ops.UINT8), (0, 2, 1))
    with pytest.raises(RmxError, match="channels-first"):
        ops.Transpose(ctx, sd, ops.desc(2, 8, 8, ops.NHWC, ops.UINT8), (2, 0, 1))
    with pytest.raises(RmxError, match="cannot hold"):
        ops.Transpose(ctx, ops.desc(2, 8, 16, ops.NHWC, ops.UINT8), ops.desc(2, 8, 16, ops.NHWC, ops.UINT8), (1, 0, 2))
