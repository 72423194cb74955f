"""rmx_resize_cmn_noalloc, the one entry point that allocates nothing (its parameter table is a static device array): two
calls in a row through the C ABI, the second with a smaller batch of smaller images, each compared bit for bit with what the
existing entry points (rmx_create_resize + rmx_update_resize_cmn + rmx_op_launch) write for the same arguments, and with the
oracle. A batch beyond the static table's rows is refused with a clear error."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops, workloads as wl
from rocal_amd._lib import RmxError

pytestmark = pytest.mark.gpu


def _case(seed, n, H, W, oh, ow):
    rng = np.random.default_rng(seed)
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.empty((n, 4), np.uint32)
    for i in range(n):
        w, h = int(rng.integers(W // 3, W + 1)), int(rng.integers(H // 3, H + 1))
        roi[i] = (int(rng.integers(0, W - w + 1)), int(rng.integers(0, H - h + 1)), w, h)
    dw = np.full(n, ow, np.uint32)
    dh = np.full(n, oh, np.uint32)
    dh[0] = oh - 3  # one ragged destination
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    scale, bias = orc.cmn_scale_bias(wl.MEAN, wl.STD, n)
    return img, roi, dw, dh, mirror, scale, bias


def test_no_alloc_entry_point_matches_the_op_entry_points_twice_in_a_row(ctx):
    import torch
    flags = ops.F_QUANTIZE_U8
    for seed, n, H, W, oh, ow in ((1, 24, 120, 160, 64, 96), (2, 7, 60, 64, 40, 48)):  # the second call: fewer, smaller images
        img, roi, dw, dh, mirror, scale, bias = _case(seed, n, H, W, oh, ow)
        sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, ops.NCHW, ops.FP16)
        src = torch.from_numpy(img).cuda()
        # the existing entry points
        op = ops.Resize(ctx, sd, dd, ops.LINEAR, flags=flags)
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        ref = op.alloc_output(fill=7)
        op.launch(src, ref)
        # the entry point that allocates nothing
        out = torch.full_like(ref, 7)
        ops.resize_cmn_noalloc(ctx, sd, dd, src, out, roi, dw, dh, scale, bias, mirror, flags=flags)
        ctx.sync()
        got, want = out.cpu().numpy(), ref.cpu().numpy()
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16)), "call with n=%d: %d values differ" % (n, int((got != want).sum()))
        exp = orc.resize(img, roi, dw, dh, oh, ow, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                         flags=orc.F_QUANTIZE_U8)
        for i in range(n):
            assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp[i, :, :dh[i], :dw[i]].view(np.uint16)), "sample %d differs from the oracle" % i
        assert (got[0, :, dh[0]:] == 7).all()  # rows below a ragged destination stay untouched


def test_no_alloc_entry_point_refuses_a_batch_beyond_its_table(ctx):
    import torch
    n = ops.NOALLOC_MAX_SAMPLES + 1
    sd, dd = ops.desc(n, 8, 8, ops.NHWC, ops.UINT8), ops.desc(n, 8, 8, ops.NCHW, ops.FP16)
    src = torch.zeros((n, 8, 8, 3), dtype=torch.uint8, device="cuda")
    dst = torch.zeros((n, 3, 8, 8), dtype=torch.float16, device="cuda")
    one = np.ones(n * 3, np.float32)
    with pytest.raises(RmxError, match="exceeds the 512 rows"):
        ops.resize_cmn_noalloc(ctx, sd, dd, src, dst, None, np.full(n, 8, np.uint32), np.full(n, 8, np.uint32), one, one)


def test_no_alloc_entry_point_can_be_captured_in_a_graph():
    """The whole call (its fill kernels carry the parameter rows as arguments) is recorded in a HIP graph and replayed on new
    pixels, with eager work and synchronisation between the replays; every replay equals the eager call."""
    import torch
    s = torch.cuda.Stream()
    c2 = ops.Context(0, stream=s.cuda_stream)
    n, H, W, oh, ow = 9, 72, 96, 40, 48
    img, roi, dw, dh, mirror, scale, bias = _case(5, n, H, W, oh, ow)
    sd, dd = ops.desc(n, H, W, ops.NHWC, ops.UINT8), ops.desc(n, oh, ow, ops.NCHW, ops.FP16)
    flags = ops.F_QUANTIZE_U8
    with torch.cuda.stream(s):
        src = torch.from_numpy(img).cuda()
        out = torch.zeros((n, 3, oh, ow), dtype=torch.float16, device="cuda")
        ops.resize_cmn_noalloc(c2, sd, dd, src, out, roi, dw, dh, scale, bias, mirror, flags=flags)  # warm-up before the capture
        s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        ops.resize_cmn_noalloc(c2, sd, dd, src, out, roi, dw, dh, scale, bias, mirror, flags=flags)
    rng = np.random.default_rng(8)
    for rep in range(4):
        pixels = rng.integers(0, 256, img.shape, dtype=np.uint8)
        with torch.cuda.stream(s):
            src.copy_(torch.from_numpy(pixels))
            out.zero_()
            g.replay()
            s.synchronize()
            got = out.cpu().numpy()
            eager = torch.zeros_like(out)
            ops.resize_cmn_noalloc(c2, sd, dd, src, eager, roi, dw, dh, scale, bias, mirror, flags=flags)
            s.synchronize()
        assert np.array_equal(got.view(np.uint16), eager.cpu().numpy().view(np.uint16)), "replay %d differs from the eager call" % rep
        exp = orc.resize(pixels, roi, dw, dh, oh, ow, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                         flags=orc.F_QUANTIZE_U8)
        for i in range(n):
            assert np.array_equal(got[i, :, :dh[i], :dw[i]].view(np.uint16), exp[i, :, :dh[i], :dw[i]].view(np.uint16)), "replay %d, sample %d" % (rep, i)
    c2.close()
