"""Parity at the full sizes of the five benchmark configurations (the CPU checker needs well under a
second for each), size-independent properties of the fused resize path, and the corner cases of the
aligned fast paths (windows that end on the last byte of the batch buffer, degenerate samples)."""
import numpy as np
import pytest

import bench
from oracle import orc
from rocal_amd import ops, workloads as wl

pytestmark = pytest.mark.gpu


def _bits(a):
    return a.view(np.uint8)


@pytest.mark.parametrize("cfg", sorted(bench.WORKLOADS))
def test_full_size_configuration_is_bit_identical_to_the_oracle(ctx, cfg):
    op, src, dst, n, cpu, _ = bench.build_case(cfg, ctx)
    dst.zero_()
    op.launch(*(src if isinstance(src, tuple) else (src,)), dst)
    ctx.sync()
    got = dst.cpu().numpy()
    exp = cpu(n)
    assert got.shape == exp.shape
    assert np.array_equal(_bits(got), _bits(exp)), "config %d: %d values differ" % (cfg, int((got != exp).sum()))


def test_fast_and_general_resize_kernels_agree_at_full_size(ctx):
    """A destination that is not 16-byte aligned sends the same batch through the general kernel."""
    import torch
    op, src, dst, n, _, _ = bench.build_case(1, ctx)
    assert "fast=1" in op.plan
    op.launch(src, dst)
    big = torch.zeros(dst.numel() + 8, dtype=dst.dtype, device="cuda")
    shifted = big[1:1 + dst.numel()].view(dst.shape)  # 2 bytes off: contiguous, unaligned
    assert shifted.data_ptr() % 16 != 0
    op.launch(src, shifted)
    ctx.sync()
    assert torch.equal(dst.view(torch.int16), shifted.view(torch.int16))


def test_mirror_is_an_involution_on_the_fused_path(ctx):
    import torch
    n = 64
    c = wl.config1(n)
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    dw = np.full(n, 224, np.uint32)
    op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
    src = torch.from_numpy(c["img"]).cuda()
    outs = []
    for mirror in (c["mirror"], 1 - c["mirror"]):
        op.update_cmn(c["roi"], dw, dw, scale, bias, mirror.astype(np.uint32))
        out = op.alloc_output()
        op.launch(src, out)
        ctx.sync()
        outs.append(out)
    assert torch.equal(outs[0].view(torch.int16), torch.flip(outs[1], dims=[3]).view(torch.int16))


def test_windows_that_end_on_the_last_bytes_of_the_batch(ctx):
    """The last sample's window reaches the last pixel of the buffer: the wide loads of the aligned
    kernels must fall back to their bounds-checked loaders there (and nowhere read past the end)."""
    import torch
    rng = np.random.default_rng(9)
    n, H, W = 3, 37, 53
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    # an exact-size allocation: nothing behind the last pixel belongs to the tensor
    src = torch.from_numpy(img.reshape(-1).copy()).cuda()
    roi = np.array([[5, 3, 48, 34], [0, 0, 53, 37], [21, 13, 32, 24]], np.uint32)  # the last two end at (52, 36)
    dw, dh = np.array([40, 64, 24], np.uint32), np.array([32, 48, 16], np.uint32)
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    mirror = np.array([1, 0, 1], np.uint32)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 48, 64, ops.NCHW, ops.FP16), ops.LINEAR)
    op.update_cmn(roi, dw, dh, scale, bias, mirror)
    assert "fast=1" in op.plan
    out = op.alloc_output()
    op.launch(src.view(n, H, W, 3), out)
    ctx.sync()
    exp = orc.resize(img, roi, dw, dh, 48, 64, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=orc.NCHW, dtype=orc.FP16)
    assert np.array_equal(_bits(out.cpu().numpy()), _bits(exp))
    # CropMirrorNormalize and ColorTwist on windows ending at the last pixel (widths multiples of 8: aligned variants)
    crop = np.array([[5, 5, 48, 32], [13, 0, 40, 37], [29, 21, 24, 16]], np.uint32)
    cmn = ops.CropMirrorNormalize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 40, 48, ops.NCHW, ops.FP32))
    cmn.update(crop, scale, bias, mirror)
    assert "fast=1" in cmn.plan
    o2 = cmn.alloc_output()
    cmn.launch(src.view(n, H, W, 3), o2)
    ctx.sync()
    e2 = orc.crop_mirror_normalize(img, crop, scale, bias, mirror, 40, 48, orc.NCHW, orc.FP32)
    assert np.array_equal(_bits(o2.cpu().numpy()), _bits(e2))
    tw = ops.ColorTwist(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 40, 48, ops.NHWC, ops.UINT8))
    one = lambda v: np.full(n, v, np.float32)
    tw.update(crop, one(1.3), one(7.0), one(40.0), one(1.4))
    o3 = tw.alloc_output()
    tw.launch(src.view(n, H, W, 3), o3)
    ctx.sync()
    sub = np.zeros((n, 40, 48, 3), np.uint8)
    full = orc.color_twist(img, np.array([[0, 0, W, H]] * n, np.uint32), one(1.3), one(7.0), one(40.0), one(1.4))
    for i, (x, y, w, h) in enumerate(crop):
        sub[i, :h, :w] = full[i, y:y + h, x:x + w]
    assert np.array_equal(o3.cpu().numpy(), sub)


def test_degenerate_samples(ctx):
    """A 1x1 source, a sample with an empty destination (skipped, output untouched) and a 1-row source."""
    import torch
    n, H, W = 3, 16, 24
    img = np.zeros((n, H, W, 3), np.uint8)
    img[0, 0, 0] = (10, 200, 77)
    img[2, 0, :, :] = np.arange(W)[:, None] * 3
    roi = np.array([[0, 0, 1, 1], [0, 0, 8, 8], [0, 0, 24, 1]], np.uint32)
    dw, dh = np.array([8, 0, 16], np.uint32), np.array([8, 8, 8], np.uint32)
    op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 8, 16, ops.NHWC, ops.UINT8), ops.LINEAR)
    op.update(roi, dw, dh)
    out = op.alloc_output(fill=9)
    op.launch(torch.from_numpy(img).cuda(), out)
    ctx.sync()
    got = out.cpu().numpy()
    exp = orc.resize(img, roi, dw, dh, 8, 16, interp=orc.LINEAR)
    assert (got[0, :8, :8] == np.array([10, 200, 77], np.uint8)).all()  # a 1x1 source is a constant image
    assert (got[1] == 9).all()                                            # nothing is written for an empty destination
    assert np.array_equal(got[0, :8, :8], exp[0, :8, :8]) and np.array_equal(got[2, :8, :16], exp[2, :8, :16])


@pytest.mark.parametrize("streaming", [False, True])
@pytest.mark.parametrize("rx,ry", [(1.3, 1.0), (1.9, 2.4), (3.0, 3.0), (3.7, 3.7), (2.5, 1.2)])
def test_triangular_downscale_tap_and_row_length_classes(ctx, rx, ry, streaming):
    """The downscaling triangular kernels: 4/6/8-tap specialisations, 1/2/3 load slots per source row, partial
    last tile, per-sample windows (edge replicas on both sides, windows away from the origin at every byte phase), mirror,
    and an exact-size source whose last rows take the bounds-checked loader. (rx, ry) are the ratios of the first sample;
    the others shrink a little more or less. streaming: a source width that is a multiple of 4 (every row starts at the
    same byte phase), which the kernel that loads rows straight into LDS takes; otherwise the one that stages through
    registers."""
    import torch
    rng = np.random.default_rng(int(rx * 100 + ry * 10))
    n, dw0, dh0 = 3, 200, 37
    W, H = int(round(dw0 * rx)) + 9, int(round(dh0 * ry)) + 5
    W = (W + 3) // 4 * 4 if streaming else W | 1
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, W - 9, H - 5], [4, 3, W - 4, H - 3], [9, 5, W - 9, H - 5]], np.uint32)  # the last two end at (W-1, H-1)
    dw = np.array([dw0, dw0 - 8, dw0 - 7], np.uint32)
    dh = np.array([dh0, dh0 - 1, dh0], np.uint32)
    mirror = np.array([0, 1, 1], np.uint32)
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    src = torch.from_numpy(img.reshape(-1).copy()).cuda()  # nothing behind the last pixel belongs to the tensor
    for dtype, layout in ((ops.FP16, ops.NCHW), (ops.UINT8, ops.NHWC)):
        op = ops.Resize(ctx, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, dh0, dw0, layout, dtype), ops.TRIANGULAR)
        if dtype == ops.UINT8:
            op.update(roi, dw, dh, mirror)
            exp = orc.resize(img, roi, dw, dh, dh0, dw0, interp=orc.TRIANGULAR, mirror=mirror, layout=layout, dtype=dtype)
        else:
            op.update_cmn(roi, dw, dh, scale, bias, mirror)
            exp = orc.resize(img, roi, dw, dh, dh0, dw0, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=layout, dtype=dtype)
        assert op.kernel_name == ("rmx_resize_tri_dma_kernel" if streaming else "rmx_resize_tri_down_kernel")
        out = op.alloc_output()
        op.launch(src.view(n, H, W, 3), out)
        ctx.sync()
        got = out.cpu().numpy()
        assert np.array_equal(_bits(got), _bits(exp)), "%d values differ" % int((got != exp).sum())


def test_triangular_ring_and_downscale_kernels_agree(ctx, monkeypatch):
    """The same downscaling batch through the ring kernel (forced), the kernel that stages rows through registers (forced)
    and the one that loads them straight into LDS."""
    import torch
    rng = np.random.default_rng(77)
    n, H, W = 2, 150, 260
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, W, H], [10, 6, 240, 140]], np.uint32)
    dw, dh = np.array([96, 88], np.uint32), np.array([64, 50], np.uint32)
    outs = []
    for ring, dma, name in (("1", "1", "rmx_resize_tri_kernel"), ("0", "0", "rmx_resize_tri_down_kernel"), ("0", "1", "rmx_resize_tri_dma_kernel")):
        monkeypatch.setenv("RMX_TUNE_TRI_RING", ring)
        monkeypatch.setenv("RMX_TUNE_DMA", dma)
        c2 = ops.Context()
        op = ops.Resize(c2, ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 64, 96, ops.NCHW, ops.FP32), ops.TRIANGULAR)
        op.update(roi, dw, dh)
        assert op.kernel_name == name
        out = op.alloc_output()
        op.launch(torch.from_numpy(img).cuda(), out)
        c2.sync()
        outs.append(out.cpu().numpy())
    assert np.array_equal(_bits(outs[0]), _bits(outs[1])) and np.array_equal(_bits(outs[0]), _bits(outs[2]))


@pytest.mark.parametrize("W", [83, 84])
@pytest.mark.parametrize("interp", [ops.LINEAR, ops.NEAREST])
def test_warp_on_an_exact_size_source_and_tiny_windows(ctx, interp, W):
    """Boxes that reach the last bytes of the batch buffer (bounds-checked staging), a 1x1 and a 2x3 ROI, ROIs away
    from the origin (repeated edge column / row), destinations that are not multiples of 8 or of the tile. Width 84: rows
    start at multiples of 4 bytes, the form of the kernel that loads boxes straight into LDS; 83: the one that stages them
    through registers."""
    import torch
    rng = np.random.default_rng(21)
    n, H = 5, 67
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.array([[0, 0, W, H], [40, 30, 1, 1], [20, 10, 2, 3], [11, 7, 72, 60], [0, 0, W, H]], np.uint32)
    dw = np.array([W, 40, 33, 77, W], np.uint32)
    dh = np.array([67, 20, 41, 50, 67], np.uint32)
    affine = np.array([[1.0, 0.0, 0.0, 1.0, 0.0, 0.0],          # identity: reads up to the last pixel
                       [0.1, 0.0, 0.0, 0.1, 0.0, 0.0],
                       [0.05, 0.02, -0.02, 0.05, 0.3, 0.2],
                       [0.9, 0.25, -0.2, 1.1, 3.5, -2.25],
                       [1.2, -0.4, 0.5, 0.8, -9.0, 12.0]], np.float32)  # rocAL order x0,y0,x1,y1,o0,o1
    m = np.stack([orc.affine_from_rocal(a) for a in affine])
    exp = orc.warp_affine(img, roi, m, dw, dh, H, W, interp=interp)
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)
    op = ops.WarpAffine(ctx, sd, sd, interp)
    op.update(roi, affine, dw, dh)
    assert op.kernel_name == ("rmx_warp_kernel(raw)" if W % 4 == 0 else "rmx_warp_kernel")
    out = op.alloc_output()
    src = torch.from_numpy(img.reshape(-1).copy()).cuda()
    op.launch(src.view(n, H, W, 3), out)
    ctx.sync()
    got = out.cpu().numpy()
    for i in range(n):
        assert np.array_equal(got[i, :dh[i], :dw[i]], exp[i, :dh[i], :dw[i]]), "sample %d: %d values differ" % (i, int((got[i, :dh[i], :dw[i]] != exp[i, :dh[i], :dw[i]]).sum()))


def test_launches_can_be_captured_in_a_graph_and_replayed(ctx):
    """update() uploads the parameter table outside the capture; the launches of a resize -> colour twist -> flip
    chain are recorded in a HIP graph and replayed several times, with eager work and synchronisation between
    the replays and a new input each time; every replay must equal the eager result. An op whose launch was recorded
    refuses further updates (its replays would read rows that the table ring hands out again)."""
    import torch
    s = torch.cuda.Stream()
    c2 = ops.Context(0, stream=s.cuda_stream)
    rng = np.random.default_rng(3)
    n, H, W = 4, 90, 120
    roi = np.array([[0, 0, 120, 90], [5, 5, 100, 80], [0, 0, 64, 64], [10, 0, 96, 90]], np.uint32)
    dw, dh = np.full(n, 64, np.uint32), np.full(n, 48, np.uint32)
    mid_roi = np.array([[0, 0, 64, 48]] * n, np.uint32)
    one = lambda v: np.full(n, v, np.float32)
    sd, md = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, 48, 64, ops.NHWC, ops.UINT8)
    resize, twist, flip = ops.Resize(c2, sd, md, ops.LINEAR), ops.ColorTwist(c2, md, md), ops.Flip(c2, md, md)
    resize.update(roi, dw, dh)
    twist.update(mid_roi, one(1.1), one(4.0), one(25.0), one(1.3))
    flip.update(mid_roi, np.ones(n, np.uint32), np.zeros(n, np.uint32))
    with torch.cuda.stream(s):
        src = torch.zeros((n, H, W, 3), dtype=torch.uint8, device="cuda")
        a, b, out = resize.alloc_output(), twist.alloc_output(), flip.alloc_output()
        resize.launch(src, a); twist.launch(a, b); flip.launch(b, out)  # warm-up before the capture
        s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        resize.launch(src, a)
        twist.launch(a, b)
        flip.launch(b, out)
    for rep in range(4):
        img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
        if rep == 2:
            # an update between replays: refused, because the graph's kernel node reads the table slot of the update before
            # the capture, which the ring would hand out again a few updates later; the replays after it are unchanged
            from rocal_amd._lib import RmxError
            for op_, args in ((resize, (roi, dw // 2, dh)), (twist, (mid_roi, one(0.9), one(1.0), one(5.0), one(1.0)))):
                with pytest.raises(RmxError, match="recorded into a HIP graph"):
                    op_.update(*args)
        with torch.cuda.stream(s):
            src.copy_(torch.from_numpy(img))
            out.zero_()
            g.replay()
            s.synchronize()
            got = out.cpu().numpy()
            # the same chain eagerly, into other buffers
            a2, b2, o2 = resize.alloc_output(), twist.alloc_output(), flip.alloc_output()
            resize.launch(src, a2); twist.launch(a2, b2); flip.launch(b2, o2)
            s.synchronize()
        exp_mid = orc.color_twist(orc.resize(img, roi, dw, dh, 48, 64, interp=orc.LINEAR), mid_roi, one(1.1), one(4.0), one(25.0), one(1.3))
        assert np.array_equal(got, o2.cpu().numpy()), "replay %d differs from the eager chain" % rep
        assert np.array_equal(got, exp_mid[:, :, ::-1]), "replay %d differs from the oracle" % rep


@pytest.mark.parametrize("layout,dtype", [(ops.NHWC, ops.FP32), (ops.NCHW, ops.FP32), (ops.NHWC, ops.FP16)])
def test_large_windows_in_narrow_tiles_every_float_format(ctx, layout, dtype):
    """RandomResizedCrop + CropMirrorNormalize from windows of up to 640 x 640 pixels: the aligned kernel narrows its x-tiles
    until a strip's window fits its LDS slice, so a row is written by several tiles; with mirrors, in every float format
    (interleaved fp32 goes through the coalescing stores)."""
    import torch
    n = 16
    c = wl.config1(n)
    c["roi"][0] = (0, 0, c["W"][0], c["H"][0])  # a whole image
    inv = (1 / wl.STD).astype(np.float32)
    scale, bias = np.tile(inv, n), np.tile(-(wl.MEAN * inv), n)
    dw = np.full(n, 224, np.uint32)
    op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, layout, dtype), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
    op.update_cmn(c["roi"], dw, dw, scale, bias, c["mirror"])
    assert op.kernel_name == ("rmx_resize_fast_kernel" if (layout, dtype) == (ops.NHWC, ops.FP32) else "rmx_resize_dma_kernel")
    out = op.alloc_output()
    op.launch(torch.from_numpy(c["img"]).cuda(), out)
    ctx.sync()
    got = out.cpu().numpy()
    exp = orc.resize(c["img"], c["roi"], dw, dw, 224, 224, interp=orc.LINEAR, mirror=c["mirror"], scale=scale, bias=bias,
                     layout=layout, dtype=dtype, flags=orc.F_QUANTIZE_U8)
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "%d values differ (%s)" % (int((got != exp).sum()), op.plan)
