"""The two aligned bilinear kernels against each other and against the oracle, bit for bit: the streaming kernel (source rows
straight into LDS) and the staged kernel (windows through registers). Covers what is specific to the streaming kernel: the
byte phases of packed pixels inside LDS rows, both edge replicas, rows cut into several x-tiles, strips of one to eight rows,
the window that ends on the last byte of the batch buffer, ragged sources and every destination format it serves."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops, workloads as wl

pytestmark = pytest.mark.gpu


def _gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _run(c, desc_src, desc_dst, flags, update, img):
    op = ops.Resize(c, desc_src, desc_dst, ops.LINEAR, flags=flags)
    update(op)
    out = op.alloc_output()
    op.launch(img, out)
    c.sync()
    return out.cpu().numpy(), op.kernel_name, op.plan


def _scale_bias(n):
    return orc.cmn_scale_bias(wl.MEAN, wl.STD, n)


@pytest.mark.parametrize("layout,dtype", [(ops.NCHW, ops.FP16), (ops.NCHW, ops.FP32), (ops.NCHW, ops.UINT8), (ops.NHWC, ops.FP16), (ops.NHWC, ops.UINT8)])
def test_streaming_and_staged_kernels_agree_with_the_oracle(ctx, ctx_staged, ctx_dma_small, layout, dtype):
    rng = np.random.default_rng(4400 + 7 * layout + dtype)
    n, H, W = 10, 150, 200  # 600-byte rows: every row starts at the same byte phase
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.empty((n, 4), np.uint32)
    for i in range(n):
        w, h = int(rng.integers(1, W + 1)), int(rng.integers(1, H + 1))
        roi[i] = (int(rng.integers(0, W - w + 1)), int(rng.integers(0, H - h + 1)), w, h)
    roi[0] = (0, 0, W, H)            # both edge replicas of the whole image
    roi[1] = (W - 9, H - 5, 9, 5)    # the window that ends on the last byte ... of sample 1
    roi[n - 1] = (W - 40, H - 30, 40, 30)  # ... and of the batch buffer: the bounds-checked staging
    roi[2] = (3, 5, 1, 1)            # a single pixel
    # ratios of at most 3 in both directions: windows that fit the smallest LDS setting in tiles of at least 8 columns
    dw = np.array([8 * int(rng.integers(-(-int(roi[i, 2]) // 24), 17)) for i in range(n)], np.uint32)
    dh = np.array([int(rng.integers(-(-int(roi[i, 3]) // 3), 100)) for i in range(n)], np.uint32)
    dw[0], dh[0] = 128, 97
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    scale, bias = _scale_bias(n)
    norm = dtype != ops.UINT8
    flags = ops.F_QUANTIZE_U8 if norm else 0
    oflags = orc.F_QUANTIZE_U8 if norm else 0
    exp = orc.resize(img, roi, dw, dh, 100, 128, interp=orc.LINEAR, mirror=mirror, scale=scale if norm else None, bias=bias if norm else None,
                     layout=layout, dtype=dtype, flags=oflags)
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 100, 128, layout, dtype)

    def update(op):
        if norm:
            op.update_cmn(roi, dw, dh, scale, bias, mirror)
        else:
            op.update(roi, dw, dh, mirror)
    dimg = _gpu(img)
    names = []
    for c in (ctx, ctx_staged, ctx_dma_small):
        got, name, plan = _run(c, sd, dd, flags, update, dimg)
        names.append(name)
        # written windows only: the rest of the padded destination keeps the fill value on both sides
        for i in range(n):
            g = got[i, :, :dh[i], :dw[i]] if layout == ops.NCHW else got[i, :dh[i], :dw[i]]
            e = exp[i, :, :dh[i], :dw[i]] if layout == ops.NCHW else exp[i, :dh[i], :dw[i]]
            assert np.array_equal(g.view(np.uint8), e.view(np.uint8)), "sample %d differs (%s, %s)" % (i, name, plan)
    assert names == ["rmx_resize_dma_kernel", "rmx_resize_fast_kernel", "rmx_resize_dma_kernel"]


@pytest.mark.parametrize("layout,dtype", [(ops.NCHW, ops.FP16), (ops.NCHW, ops.FP32), (ops.NCHW, ops.UINT8), (ops.NHWC, ops.FP16),
                                          (ops.NHWC, ops.FP32), (ops.NHWC, ops.UINT8)])
def test_streaming_kernel_any_width_and_any_destination_base(ctx, ctx_dma_small, layout, dtype):
    """Destination widths that are not multiples of 8 (225, 37, 1 ...) and a destination whose first byte is not 16-byte
    aligned: the streaming kernel's any-width form stores element by element. Every format, interleaved fp32 included; short
    last groups of every length 1..7; mirrored and unmirrored; tiles cut by the small LDS setting; the padding around each
    written window must keep the fill value."""
    import torch
    rng = np.random.default_rng(5100 + 7 * layout + dtype)
    n, H, W = 12, 150, 200
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.empty((n, 4), np.uint32)
    for i in range(n):
        w, h = int(rng.integers(1, W + 1)), int(rng.integers(1, H + 1))
        roi[i] = (int(rng.integers(0, W - w + 1)), int(rng.integers(0, H - h + 1)), w, h)
    roi[0] = (0, 0, W, H)
    roi[1] = (W - 9, H - 5, 9, 5)
    roi[n - 1] = (W - 40, H - 30, 40, 30)  # ends on the last byte of the batch buffer
    roi[2] = (3, 5, 1, 1)
    OH, OW = 100, 229
    dw = np.array([int(rng.integers(max(1, -(-int(roi[i, 2]) // 3)), OW + 1)) for i in range(n)], np.uint32)
    dh = np.array([int(rng.integers(max(1, -(-int(roi[i, 3]) // 3)), OH + 1)) for i in range(n)], np.uint32)
    dw[0], dh[0] = 225, 97
    dw[2] = 1
    dw[3:10] = 8 * (dw[3:10] // 8) + np.arange(1, 8)  # every length of the short last group
    dw = np.minimum(dw, OW).astype(np.uint32)
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    mirror[0] = 1
    scale, bias = _scale_bias(n)
    norm = dtype != ops.UINT8
    flags = ops.F_QUANTIZE_U8 if norm else 0
    exp = orc.resize(img, roi, dw, dh, OH, OW, interp=orc.LINEAR, mirror=mirror, scale=scale if norm else None, bias=bias if norm else None,
                     layout=layout, dtype=dtype, flags=orc.F_QUANTIZE_U8 if norm else 0)
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, layout, dtype)
    dimg = _gpu(img)
    esz = exp.dtype.itemsize
    for c in (ctx, ctx_dma_small):
        op = ops.Resize(c, sd, dd, ops.LINEAR, flags=flags)
        if norm:
            op.update_cmn(roi, dw, dh, scale, bias, mirror)
        else:
            op.update(roi, dw, dh, mirror)
        assert op.kernel_name == "rmx_resize_dma_kernel" and "any_width=1" in op.plan, op.plan
        for shift in (0, 1, 3):  # elements between a 256-byte boundary and the destination's first byte
            raw = torch.full((exp.size * esz + 256,), 0x5A, dtype=torch.uint8, device="cuda")
            out = raw[shift * esz: shift * esz + exp.size * esz].view(ops.torch_dtype(dtype)).view(exp.shape)
            op.launch(dimg, out)
            c.sync()
            got = out.cpu().numpy()
            fill = np.frombuffer(bytes([0x5A]) * esz, exp.dtype)[0]
            want = np.full_like(exp, fill)
            for i in range(n):
                if layout == ops.NCHW:
                    want[i, :, :dh[i], :dw[i]] = exp[i, :, :dh[i], :dw[i]]
                else:
                    want[i, :dh[i], :dw[i]] = exp[i, :dh[i], :dw[i]]
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), "shift %d (%s)" % (shift, op.plan)
            r = raw.cpu().numpy()
            assert (r[:shift * esz] == 0x5A).all() and (r[shift * esz + exp.size * esz:] == 0x5A).all()


@pytest.mark.parametrize("rows", [1, 3, 4, 8])
def test_strip_heights(rows):
    """Strips of one to eight rows, with destination heights that leave a short last strip."""
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_FAST_ROWS=rows)
    rng = np.random.default_rng(99)
    n, H, W = 6, 96, 128
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    roi = np.array([[0, 0, 128, 96], [7, 9, 100, 80], [0, 0, 64, 96], [20, 20, 31, 17], [1, 0, 127, 96], [0, 3, 128, 90]], np.uint32)
    dw = np.array([64, 128, 8, 72, 128, 96], np.uint32)
    dh = np.array([61, 1, 47, 4, 96, 5], np.uint32)
    mirror = np.array([0, 1, 1, 0, 1, 0], np.uint32)
    scale, bias = _scale_bias(n)
    exp = orc.resize(img, roi, dw, dh, 96, 128, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                     flags=orc.F_QUANTIZE_U8)
    got, name, plan = _run(c, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 96, 128, ops.NCHW, ops.FP16), ops.F_QUANTIZE_U8,
                           lambda op: op.update_cmn(roi, dw, dh, scale, bias, mirror), _gpu(img))
    assert name == "rmx_resize_dma_kernel" and ("strip_rows=%d " % rows) in plan, plan
    for i in range(n):
        assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp[i, :, :dh[i], :dw[i]].view(np.uint16)), "sample %d (%s)" % (i, plan)
    c.close()


def test_ragged_source_with_dword_row_strides(ctx):
    """Tightly packed images whose widths are multiples of 4 (row strides multiples of 4 bytes, bases at any dword): the streaming
    kernel; one odd width sends the batch to the staged kernel. Same results."""
    rng = np.random.default_rng(5)
    n = 6
    widths = np.array([64, 100, 36, 128, 88, 12], np.uint32)
    heights = np.array([50, 33, 80, 64, 21, 9], np.uint32)
    for odd in (False, True):
        w = widths.copy()
        if odd:
            w[2] = 37
        imgs = [rng.integers(0, 256, (int(heights[i]), int(w[i]), 3), dtype=np.uint8) for i in range(n)]
        offsets, pos, parts = [], 0, []
        for im in imgs:
            pad = (-pos) % 4  # images start at dword addresses
            parts.append(np.zeros(pad, np.uint8))
            pos += pad
            offsets.append(pos)
            parts.append(im.reshape(-1))
            pos += im.size
        packed = np.concatenate(parts)
        padded = np.zeros((n, 80, 128, 3), np.uint8)
        for i, im in enumerate(imgs):
            padded[i, :im.shape[0], :im.shape[1]] = im
        roi = np.array([[0, 0, w[i], heights[i]] for i in range(n)], np.uint32)
        roi[1] = (10, 5, 80, 20)
        dw = np.array([48, 64, 40, 128, 8, 24], np.uint32)
        dh = np.array([40, 30, 90, 50, 30, 18], np.uint32)
        mirror = np.array([1, 0, 0, 1, 1, 0], np.uint32)
        scale, bias = _scale_bias(n)
        exp = orc.resize(padded, roi, dw, dh, 90, 128, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                         flags=orc.F_QUANTIZE_U8)
        op = ops.Resize(ctx, ops.desc(n, 80, 128, ops.NHWC, ops.UINT8), ops.desc(n, 90, 128, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
        op.set_ragged_source(np.array(offsets, np.uint64), w, heights, packed.size)
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        assert op.kernel_name == ("rmx_resize_fast_kernel" if odd else "rmx_resize_dma_kernel")
        out = op.alloc_output()
        op.launch(_gpu(packed), out)
        ctx.sync()
        got = out.cpu().numpy()
        for i in range(n):
            assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp[i, :, :dh[i], :dw[i]].view(np.uint16)), "sample %d, odd=%s" % (i, odd)


def test_ragged_source_with_padded_rows(ctx):
    """Packed images of any width whose rows the loader pads to a multiple of 4 bytes (a row stride per image): the streaming
    kernel, bit-identical to the oracle on the padded tensor; a stride shorter than a row is refused."""
    rng = np.random.default_rng(6)
    n = 6
    widths = np.array([61, 100, 37, 127, 85, 11], np.uint32)
    heights = np.array([50, 33, 80, 64, 21, 9], np.uint32)
    strides = (3 * widths + 3) // 4 * 4
    offsets, parts, pos = [], [], 0
    padded = np.zeros((n, 80, 128, 3), np.uint8)
    for i in range(n):
        h, w, st = int(heights[i]), int(widths[i]), int(strides[i])
        im = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
        padded[i, :h, :w] = im
        rows = rng.integers(0, 256, (h, st), dtype=np.uint8)  # the padding bytes hold anything
        rows[:, :3 * w] = im.reshape(h, 3 * w)
        offsets.append(pos)
        parts.append(rows.reshape(-1))
        pos += h * st
    packed = np.concatenate(parts)
    roi = np.array([[0, 0, widths[i], heights[i]] for i in range(n)], np.uint32)
    roi[1] = (10, 5, 80, 20)
    dw = np.array([48, 64, 40, 128, 8, 24], np.uint32)
    dh = np.array([40, 30, 90, 50, 30, 18], np.uint32)
    mirror = np.array([1, 0, 0, 1, 1, 0], np.uint32)
    scale, bias = _scale_bias(n)
    exp = orc.resize(padded, roi, dw, dh, 90, 128, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                     flags=orc.F_QUANTIZE_U8)
    op = ops.Resize(ctx, ops.desc(n, 80, 128, ops.NHWC, ops.UINT8), ops.desc(n, 90, 128, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
    op.set_ragged_source(np.array(offsets, np.uint64), widths, heights, packed.size, row_strides=strides)
    op.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert op.kernel_name == "rmx_resize_dma_kernel"
    out = op.alloc_output()
    op.launch(_gpu(packed), out)
    ctx.sync()
    got = out.cpu().numpy()
    for i in range(n):
        assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp[i, :, :dh[i], :dw[i]].view(np.uint16)), "sample %d" % i
    with pytest.raises(Exception, match="row stride"):
        op.set_ragged_source(np.array(offsets, np.uint64), widths, heights, packed.size, row_strides=3 * widths - 1)
    # windows are clipped to the image, not to the padded row: image 2 is 37 pixels wide in rows of 112 bytes (37.3 pixels)
    op.set_ragged_source(np.array(offsets, np.uint64), widths, heights, packed.size, row_strides=strides)
    wide = roi.copy()
    wide[:, 2] = 1000
    op.update_cmn(wide, dw, dh, scale, bias, mirror)
    op.launch(_gpu(packed), out)
    ctx.sync()
    full = np.array([[0, 0, widths[i], heights[i]] for i in range(n)], np.uint32)
    full[1] = (10, 5, widths[1] - 10, 20)
    exp2 = orc.resize(padded, full, dw, dh, 90, 128, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                      flags=orc.F_QUANTIZE_U8)
    got = out.cpu().numpy()
    for i in range(n):
        assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp2[i, :, :dh[i], :dw[i]].view(np.uint16)), "clipped window, sample %d" % i
