"""The streaming triangular kernel (source rows straight into LDS as packed bytes) against the oracle, bit for bit, on what is
specific to it: windows that start at every byte phase of a dword, edge replicas on both sides, every output format, strips
whose source rows outnumber the table of vertical coefficients, many vertical taps, mirror, packed (ragged) sources whose
rows start at multiples of 4 bytes (image bases at every byte phase), and the kernel that stages through registers on the same
batches; the same packed sources through the raw form of the warp kernel."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops, workloads as wl

pytestmark = pytest.mark.gpu


def _gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint8)


def _scale_bias(n):
    return orc.cmn_scale_bias(wl.MEAN, wl.STD, n)


def _check_windows(got, exp, dw, dh, layout, fill, what):
    n = got.shape[0]
    want = np.full_like(exp, fill)
    for i in range(n):
        if layout == ops.NCHW:
            want[i, :, :dh[i], :dw[i]] = exp[i, :, :dh[i], :dw[i]]
        else:
            want[i, :dh[i], :dw[i]] = exp[i, :dh[i], :dw[i]]
    assert np.array_equal(_bits(got), _bits(want)), "%s: %d values differ" % (what, int((got != want).sum()))


@pytest.mark.parametrize("layout,dtype", [(ops.NCHW, ops.FP16), (ops.NCHW, ops.FP32), (ops.NCHW, ops.UINT8), (ops.NHWC, ops.FP16),
                                          (ops.NHWC, ops.FP32), (ops.NHWC, ops.UINT8)])
def test_formats_phases_and_edges(ctx, ctx_staged, layout, dtype):
    """Eight samples over a 256-pixel-wide source (768-byte rows): the whole image (replicas left and right), windows whose
    first column is 1, 2, 3 ... pixels in (every byte phase), windows that end at the last column / row, a narrow and a
    short one; destinations narrower than the tensor (the padding keeps the fill value); both kernels."""
    rng = np.random.default_rng(900 + 7 * layout + dtype)
    n, H, W = 8, 200, 256
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, W, H], [1, 0, 200, 150], [2, 7, 222, 180], [3, 1, 253, 199], [5, 9, 251, 191], [40, 30, 60, 90], [100, 150, 156, 50],
                    [0, 0, W, H]], np.uint32)
    dw = np.array([100, 77, 129, 64, 130, 31, 57, 200], np.uint32)
    dh = np.array([61, 50, 47, 30, 61, 40, 11, 61], np.uint32)
    OH, OW = 61, 200
    mirror = np.array([0, 1, 0, 1, 1, 0, 1, 0], np.uint32)
    scale, bias = _scale_bias(n)
    norm = dtype != ops.UINT8
    exp = orc.resize(img, roi, dw, dh, OH, OW, interp=orc.TRIANGULAR, mirror=mirror, scale=scale if norm else None, bias=bias if norm else None,
                     layout=layout, dtype=dtype)
    for c, name in ((ctx, "rmx_resize_tri_dma_kernel"), (ctx_staged, "rmx_resize_tri_down_kernel")):
        op = ops.Resize(c, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, layout, dtype), ops.TRIANGULAR)
        if norm:
            op.update_cmn(roi, dw, dh, scale, bias, mirror)
        else:
            op.update(roi, dw, dh, mirror)
        assert op.kernel_name == name, op.plan
        out = op.alloc_output(fill=7)
        op.launch(_gpu(img), out)
        c.sync()
        _check_windows(out.cpu().numpy(), exp, dw, dh, layout, 7, name)


@pytest.mark.parametrize("ry,rows", [(7.4, 0), (5.1, 20), (2.0, 64), (1.0, 7)])
def test_many_vertical_taps_and_long_strips(ctx, ry, rows):
    """Vertical ratios up to 7.4 (15 taps: rows at the window's ends are read by up to 8 clamped taps each), strips whose
    source rows outnumber the 64 rows of the coefficient table (it is rebuilt on the way), strips of 64 output rows, ratio 1."""
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_TRI_ROWS=rows) if rows else ctx
    rng = np.random.default_rng(int(ry * 10) + rows)
    n, dh0, dw0 = 3, 70, 150
    H, W = int(round(dh0 * ry)) + 6, 340
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    roi = np.array([[0, 0, W, H], [4, 3, 300, H - 6], [17, 0, 323, H - 1]], np.uint32)
    dw = np.array([dw0, 131, 150], np.uint32)
    dh = np.array([dh0, dh0 - 3, dh0], np.uint32)
    mirror = np.array([1, 0, 1], np.uint32)
    scale, bias = _scale_bias(n)
    exp = orc.resize(img, roi, dw, dh, dh0, dw0, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16)
    op = ops.Resize(c, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, dh0, dw0, ops.NCHW, ops.FP16), ops.TRIANGULAR)
    op.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert op.kernel_name == "rmx_resize_tri_dma_kernel", op.plan
    out = op.alloc_output(fill=3)
    op.launch(_gpu(img), out)
    c.sync()
    _check_windows(out.cpu().numpy(), exp, dw, dh, ops.NCHW, 3, "ry=%g rows=%d (%s)" % (ry, rows, op.plan))
    if rows:
        c.close()


@pytest.fixture(scope="module")
def ctx_four_rows():
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_TRI_SLOTS=4)
    yield c
    c.close()


@pytest.mark.parametrize("ry", [1.0, 1.5, 2.0, 2.5, 3.0, 4.0, 6.5])
@pytest.mark.parametrize("rows", [0, 5])
def test_whole_and_half_ratios_keep_two_rows_in_flight(ctx, ctx_four_rows, ry, rows):
    """Vertical ratios that are whole or half numbers: output rows two apart never share a source row, the kernel keeps two
    accumulator sets instead of four. Windows at the top, in the middle and at the bottom of the source (the clamp at either
    end), a window of two output rows, mirror, strips of five rows and planned ones; against the oracle and, bit for bit,
    against the four-row form. A sample of another ratio in the batch sends the whole batch to the four-row form."""
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_TRI_ROWS=rows) if rows else ctx
    rng = np.random.default_rng(int(ry * 10) + rows)
    n, OH, OW = 5, 60, 140
    H, W = int(OH * ry) + 48, 300
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    dh = np.array([OH, 52, 34, 2, OH], np.uint32)  # even heights: the source heights below are whole numbers for half ratios too
    dw = np.array([OW, 131, 140, 60, 99], np.uint32)
    sh = np.array([int(d * ry) for d in dh], np.uint32)
    assert all(float(s) / float(d) == ry for s, d in zip(sh, dh))
    roi = np.array([[0, 0, W, sh[0]], [4, 17, 280, sh[1]], [16, H - sh[2], 284, sh[2]], [1, 9, 200, sh[3]], [0, 40, 250, sh[4]]], np.uint32)
    mirror = np.array([1, 0, 1, 0, 0], np.uint32)
    scale, bias = _scale_bias(n)
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, ops.NCHW, ops.FP16)
    exp = orc.resize(img, roi, dw, dh, OH, OW, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16)
    src = _gpu(img)
    op = ops.Resize(c, sd, dd, ops.TRIANGULAR)
    op.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert op.kernel_name == "rmx_resize_tri_dma_kernel" and "rows_in_flight=2" in op.plan, op.plan
    out = op.alloc_output(fill=3)
    op.launch(src, out)
    c.sync()
    _check_windows(out.cpu().numpy(), exp, dw, dh, ops.NCHW, 3, "ry=%g (%s)" % (ry, op.plan))
    op4 = ops.Resize(ctx_four_rows, sd, dd, ops.TRIANGULAR)
    op4.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert "rows_in_flight=4" in op4.plan, op4.plan
    out4 = op4.alloc_output(fill=3)
    op4.launch(src, out4)
    ctx_four_rows.sync()
    assert np.array_equal(_bits(out.cpu().numpy()), _bits(out4.cpu().numpy()))
    # one window of another ratio: four rows in flight for the batch, same results for the others
    roi2, dh2 = roi.copy(), dh.copy()
    roi2[4, 3] = sh[4] + 3
    exp2 = orc.resize(img, roi2, dw, dh2, OH, OW, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16)
    op.update_cmn(roi2, dw, dh2, scale, bias, mirror)
    assert "rows_in_flight=4" in op.plan, op.plan
    out2 = op.alloc_output(fill=3)
    op.launch(src, out2)
    c.sync()
    _check_windows(out2.cpu().numpy(), exp2, dw, dh2, ops.NCHW, 3, "mixed ratios (%s)" % op.plan)
    if rows:
        c.close()


@pytest.mark.parametrize("seed", range(6))
def test_random_whole_and_half_ratios_with_a_crop_behind_the_resize(ctx, seed):
    """Seeded sweep of the two-row form: per sample a vertical ratio k / 2 (k = 2 .. 12), any horizontal ratio between 1 and 4,
    a window anywhere in the source, and a crop window inside the resized image (the strip's first output row is then not the
    image's first), fused resize -> quantise -> crop -> mirror -> normalise against the two oracle nodes."""
    rng = np.random.default_rng(7000 + seed)
    n = int(rng.integers(2, 7))
    k = rng.integers(2, 13, n)
    dh = (rng.integers(4, 31, n) * 2).astype(np.uint32)          # even: the source height k dh / 2 is a whole number
    sh = (dh.astype(np.int64) * k // 2).astype(np.uint32)
    dw = rng.integers(16, 151, n).astype(np.uint32)
    sw = np.array([int(rng.integers(d, min(4 * d, 400) + 1)) for d in dw], np.uint32)
    y0 = rng.integers(0, 20, n).astype(np.uint32)
    x0 = rng.integers(0, 20, n).astype(np.uint32)
    H, W = int((y0 + sh).max()) + int(rng.integers(0, 5)), (int((x0 + sw).max()) + 3) // 4 * 4
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    roi = np.stack([x0, y0, sw, sh], 1).astype(np.uint32)
    crop = np.empty((n, 4), np.uint32)
    for i in range(n):
        cw, ch = int(rng.integers(1, dw[i] + 1)), int(rng.integers(1, dh[i] + 1))
        crop[i] = (int(rng.integers(0, dw[i] - cw + 1)), int(rng.integers(0, dh[i] - ch + 1)), cw, ch)
    OH, OW = int(crop[:, 3].max()), int(crop[:, 2].max())
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    scale, bias = _scale_bias(n)
    mid = orc.resize(img, roi, dw, dh, int(dh.max()), int(dw.max()), interp=orc.TRIANGULAR)
    exp = orc.crop_mirror_normalize(mid, crop, scale, bias, mirror, OH, OW, ops.NCHW, ops.FP32)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, ops.NCHW, ops.FP32), ops.TRIANGULAR, flags=ops.F_QUANTIZE_U8)
    op.update_cmn(roi, dw, dh, scale, bias, mirror, crop_roi=crop)
    assert op.kernel_name == "rmx_resize_tri_dma_kernel" and "rows_in_flight=2" in op.plan, op.plan
    out = op.alloc_output(fill=5)
    op.launch(_gpu(img), out)
    ctx.sync()
    _check_windows(out.cpu().numpy(), exp, crop[:, 2], crop[:, 3], ops.NCHW, 5, "seed %d (%s)" % (seed, op.plan))


@pytest.mark.parametrize("rx,layout,dtype", [(1, ops.NCHW, ops.FP16), (2, ops.NCHW, ops.FP16), (3, ops.NCHW, ops.FP16), (5, ops.NCHW, ops.FP16),
                                             (2, ops.NHWC, ops.UINT8), (3, ops.NHWC, ops.FP32)])
def test_whole_horizontal_ratios(ctx, ctx_staged, rx, layout, dtype):
    """Horizontal ratios 1 and 3: the first tap of every column has coefficient 0 and the streaming kernel runs one tap less
    (1 and 5 taps: its 4- and 5-tap passes); ratio 5 has ten taps and goes to the ring kernel. Ratios 2 and 3: a lane takes two
    NEIGHBOURING columns and reads the union of their taps once (rows of even width: 150 = a tile of 128 and one of 22, and 140;
    the row of 31 columns keeps the columns 64 apart). Windows at the left and right end of the source (replicas), in the
    middle, mirrored; a second tile (more than 128 columns); a batch with one window of another ratio, whose wavefronts keep
    the first tap and the columns apart. Against the oracle, also through the kernel that stages through registers."""
    rng = np.random.default_rng(50 + rx)
    n, OH, OW = 4, 24, 150
    dw = np.array([OW, 140, 31, 150], np.uint32)
    sw = (dw * rx).astype(np.uint32)
    sw[3] = sw[3] + 2                                   # ratio (150 rx + 2) / 150: first taps with coefficients
    W = (int(sw.max()) + 11) // 4 * 4
    H = 60
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    roi = np.array([[0, 0, sw[0], 48], [W - sw[1], 5, sw[1], 50], [7, 3, sw[2], 36], [1, 0, sw[3], 60]], np.uint32)
    dh = np.array([OH, 20, 18, 24], np.uint32)
    mirror = np.array([0, 1, 0, 1], np.uint32)
    scale, bias = _scale_bias(n)
    norm = dtype != ops.UINT8
    kw = dict(interp=orc.TRIANGULAR, mirror=mirror, scale=scale if norm else None, bias=bias if norm else None, layout=layout, dtype=dtype)
    exp = orc.resize(img, roi, dw, dh, OH, OW, **kw)
    for c in (ctx, ctx_staged):
        op = ops.Resize(c, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, layout, dtype), ops.TRIANGULAR)
        if norm:
            op.update_cmn(roi, dw, dh, scale, bias, mirror)
        else:
            op.update(roi, dw, dh, mirror)
        if c is ctx:
            assert op.kernel_name == ("rmx_resize_tri_dma_kernel" if rx < 5 else "rmx_resize_tri_kernel"), op.plan
        out = op.alloc_output(fill=9)
        op.launch(_gpu(img), out)
        c.sync()
        _check_windows(out.cpu().numpy(), exp, dw, dh, layout, 9, "rx=%d %s" % (rx, op.kernel_name))


@pytest.mark.parametrize("layout,dtype", [(ops.NCHW, ops.FP16), (ops.NHWC, ops.UINT8), (ops.NCHW, ops.FP32)])
@pytest.mark.parametrize("rows", [0, 7])
def test_windows_that_grow_keep_eight_rows_in_flight(ctx, ctx_four_rows, layout, dtype, rows):
    """A batch of windows some of which shrink and some of which grow (vertical ratios 0.28 .. 2.6, as RandomResizedCrop makes
    them): the streaming kernel keeps eight output rows in flight. Windows at the top and at the bottom of the source (the
    clamp), mirrored, growing in one direction and shrinking in the other; against the oracle and, bit for bit, against the
    ring kernel. A window that grows by more than the eight rows allow sends the batch to the ring kernel."""
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_TRI_ROWS=rows) if rows else ctx
    rng = np.random.default_rng(8100 + 10 * layout + dtype + rows)
    n, H, W, OH, OW = 7, 160, 200, 64, 96
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    roi = np.array([[0, 0, W, H], [4, 0, 40, 18], [100, H - 23, 96, 23], [8, 30, 150, 29], [0, 100, 30, 60], [60, 0, 131, 58], [20, 10, 27, 150]], np.uint32)
    dw = np.array([OW, 96, 88, 41, 96, 96, 80], np.uint32)
    dh = np.array([OH, 64, 64, 64, 57, 64, 58], np.uint32)    # vertical ratios 2.5, 0.28, 0.36, 0.45, 1.05, 0.91, 2.59
    mirror = np.array([0, 1, 0, 1, 1, 0, 1], np.uint32)
    scale, bias = _scale_bias(n)
    norm = dtype != ops.UINT8
    kw = dict(interp=orc.TRIANGULAR, mirror=mirror, scale=scale if norm else None, bias=bias if norm else None, layout=layout, dtype=dtype)
    exp = orc.resize(img, roi, dw, dh, OH, OW, **kw)
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, layout, dtype)
    src = _gpu(img)

    def run(cx, r, h):
        op = ops.Resize(cx, sd, dd, ops.TRIANGULAR)
        if norm:
            op.update_cmn(r, dw, h, scale, bias, mirror)
        else:
            op.update(r, dw, h, mirror)
        out = op.alloc_output(fill=4)
        op.launch(src, out)
        cx.sync()
        return op, out.cpu().numpy()

    op, got = run(c, roi, dh)
    assert op.kernel_name == "rmx_resize_tri_dma_kernel" and "rows_in_flight=8" in op.plan, op.plan
    _check_windows(got, exp, dw, dh, layout, 4, "eight rows (%s)" % op.plan)
    op4, got4 = run(ctx_four_rows, roi, dh)
    assert op4.kernel_name == "rmx_resize_tri_kernel", op4.plan
    assert np.array_equal(_bits(got), _bits(got4))
    roi2 = roi.copy()
    roi2[1, 3] = 12                                            # 12 rows to 64: ratio 0.19
    op2, got2 = run(c, roi2, dh)
    assert op2.kernel_name == "rmx_resize_tri_kernel", op2.plan
    _check_windows(got2, orc.resize(img, roi2, dw, dh, OH, OW, **kw), dw, dh, layout, 4, "ring kernel")
    if rows:
        c.close()


def test_more_than_sixteen_vertical_taps_take_the_other_kernel(ctx):
    rng = np.random.default_rng(3)
    n, H, W = 1, 400, 64
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, W, H]], np.uint32)
    dw, dh = np.array([32], np.uint32), np.array([40], np.uint32)  # ratio 10: 20 taps
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 40, 32, ops.NHWC, ops.UINT8), ops.TRIANGULAR)
    op.update(roi, dw, dh)
    assert op.kernel_name == "rmx_resize_tri_down_kernel"
    out = op.alloc_output()
    op.launch(_gpu(img), out)
    ctx.sync()
    exp = orc.resize(img, roi, dw, dh, 40, 32, interp=orc.TRIANGULAR, layout=ops.NHWC, dtype=ops.UINT8)
    assert np.array_equal(out.cpu().numpy(), exp)


def _packed(rng, widths, heights, gaps):
    """Images packed into one buffer, rows padded to multiples of 4 bytes, `gaps[i]` bytes in front of image i (so that image
    bases fall on every byte phase); returns (buffer, offsets, strides, the same images in a padded tensor)."""
    n = len(widths)
    strides = (3 * widths + 3) // 4 * 4
    offsets, parts, pos = [], [], 0
    padded = np.zeros((n, int(heights.max()), int(widths.max()), 3), np.uint8)
    for i in range(n):
        h, w, st = int(heights[i]), int(widths[i]), int(strides[i])
        im = rng.integers(0, 256, (h, w, 3), dtype=np.uint8)
        padded[i, :h, :w] = im
        rows = np.zeros((h, st), np.uint8)
        rows[:, :3 * w] = im.reshape(h, 3 * w)
        parts.append(np.full(int(gaps[i]), 0xEE, np.uint8))
        pos += int(gaps[i])
        offsets.append(pos)
        parts.append(rows.reshape(-1))
        pos += rows.size
    packed = np.concatenate(parts)
    packed = packed[:offsets[-1] + (int(heights[-1]) - 1) * int(strides[-1]) + 3 * int(widths[-1])]  # nothing behind the last pixel
    return packed, np.array(offsets, np.uint64), strides.astype(np.uint32), padded


@pytest.mark.parametrize("heights_out", [(50, 40, 31, 60), (60, 60, 60, 20)])
def test_packed_source_with_rows_at_multiples_of_four(ctx, heights_out):
    """Packed images (a byte offset and a row stride per image, strides multiples of 4, bases at byte phases 0, 1, 2, 3) in an
    exact-size buffer: the last rows of the last image end on the last bytes of the buffer and are staged by the lanes with
    bounds-checked loads. The second set of output heights makes the vertical ratios differ by more than 1.5 (2.0 .. 7.5): the
    table rows of such a batch go to the device largest window first, each naming its sample."""
    rng = np.random.default_rng(8)
    n = 4
    widths = np.array([300, 257, 128, 400], np.uint32)
    heights = np.array([120, 90, 77, 150], np.uint32)
    packed, offsets, strides, padded = _packed(rng, widths, heights, [0, 1, 2, 3])
    assert sorted(int(o) % 4 for o in offsets) == [0, 1, 2, 3] or len(set(int(o) % 4 for o in offsets)) >= 3
    roi = np.array([[0, 0, widths[i], heights[i]] for i in range(n)], np.uint32)
    roi[1] = (3, 2, 250, 85)
    dw = np.array([140, 100, 64, 180], np.uint32)
    dh = np.array(heights_out, np.uint32)
    mirror = np.array([0, 1, 1, 0], np.uint32)
    scale, bias = _scale_bias(n)
    exp = orc.resize(padded, roi, dw, dh, 60, 180, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16)
    op = ops.Resize(ctx, ops.desc(n, 150, 400, ops.NHWC, ops.UINT8), ops.desc(n, 60, 180, ops.NCHW, ops.FP16), ops.TRIANGULAR)
    op.set_ragged_source(offsets, widths, heights, packed.size, row_strides=strides)
    op.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert op.kernel_name == "rmx_resize_tri_dma_kernel", op.plan
    # (torch places the buffer at a 256-byte boundary; the kernels require a 4-byte aligned buffer, not aligned images)
    out = op.alloc_output(fill=1)
    op.launch(_gpu(packed), out)
    ctx.sync()
    _check_windows(out.cpu().numpy(), exp, dw, dh, ops.NCHW, 1, "packed source")


@pytest.mark.parametrize("interp", [ops.LINEAR, ops.NEAREST])
def test_warp_on_a_packed_source_with_rows_at_multiples_of_four(ctx, interp):
    """The same kind of source through WarpAffine: its form that loads source boxes straight into LDS, with image bases at
    every byte phase and boxes that end on the last bytes of the buffer."""
    rng = np.random.default_rng(9)
    n = 4
    widths = np.array([120, 97, 64, 150], np.uint32)
    heights = np.array([90, 70, 33, 110], np.uint32)
    packed, offsets, strides, padded = _packed(rng, widths, heights, [0, 3, 2, 1])
    H, W = padded.shape[1], padded.shape[2]
    roi = np.array([[0, 0, widths[i], heights[i]] for i in range(n)], np.uint32)
    roi[1] = (5, 4, 80, 60)
    affine = np.array([[1.0, 0.0, 0.0, 1.0, 0.0, 0.0], [0.9, 0.25, -0.2, 1.1, 3.5, -2.25], [0.7, -0.6, 0.6, 0.7, 1.0, 2.0], [1.0, 0.0, 0.0, 1.0, 0.4, 0.6]], np.float32)
    dw = np.array([120, 80, 64, 150], np.uint32)
    dh = np.array([90, 60, 33, 110], np.uint32)
    m = np.stack([orc.affine_from_rocal(a) for a in affine])
    exp = orc.warp_affine(padded, roi, m, dw, dh, H, W, interp=interp)
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)
    op = ops.WarpAffine(ctx, sd, sd, interp)
    op.set_ragged_source(offsets, widths, heights, packed.size, row_strides=strides)
    op.update(roi, affine, dw, dh)
    assert op.kernel_name == "rmx_warp_kernel(raw)", op.plan
    out = op.alloc_output()
    op.launch(_gpu(packed), out)
    ctx.sync()
    got = out.cpu().numpy()
    for i in range(n):
        assert np.array_equal(got[i, :dh[i], :dw[i]], exp[i, :dh[i], :dw[i]]), "sample %d: %d values differ" % (i, int((got[i, :dh[i], :dw[i]] != exp[i, :dh[i], :dw[i]]).sum()))


def test_rows_in_another_order_with_an_empty_sample(ctx):
    """A batch of uneven cost (vertical ratios 0.6 .. 3, so its table rows go to the device largest window first) in which one
    sample has an empty destination: that sample's output stays untouched wherever its row ends up, the others match the
    oracle, and a second update of the same op with other windows (another order) does too."""
    rng = np.random.default_rng(77)
    n, H, W, OH, OW = 5, 96, 100, 32, 32
    img = wl.smooth_noise(rng, n, H, W, sigma=1.0)
    scale, bias = _scale_bias(n)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, OH, OW, ops.NCHW, ops.FP16), ops.TRIANGULAR)
    src = _gpu(img)
    for roi in ([[0, 0, 64, 64], [3, 5, 40, 40], [10, 10, 20, 20], [0, 0, 50, 50], [2, 1, 96, 90]],
                [[1, 1, 20, 19], [0, 0, 100, 96], [7, 9, 33, 41], [0, 0, 50, 50], [5, 5, 64, 60]]):
        roi = np.array(roi, np.uint32)
        dw = np.array([32, 32, 32, 0, 32], np.uint32)
        dh = np.array([32, 32, 32, 32, 30], np.uint32)
        mirror = np.array([1, 0, 0, 1, 0], np.uint32)
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        assert op.kernel_name == "rmx_resize_tri_dma_kernel" and "rows_in_flight=8" in op.plan, op.plan
        out = op.alloc_output(fill=5)
        op.launch(src, out)
        ctx.sync()
        exp = orc.resize(img, roi, np.maximum(dw, 1), dh, OH, OW, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16)
        _check_windows(out.cpu().numpy(), exp, dw, dh, ops.NCHW, 5, "sorted rows")
