"""Which wavefront works on which sample: the kernels deal the samples round-robin to the XCDs (sample 8 i + k is the i-th
sample of XCD k) for batches of 16 samples and more; samples behind the last full round of eight keep their place. Batch sizes
that are and are not multiples of 8, distinct parameters per sample (a sample handled under another's row would show), several
kernel families, against the oracle and against a context with the deal switched off."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import ops, workloads as wl

pytestmark = pytest.mark.gpu


def _gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def ctx_batch_order():
    from conftest import _ctx_with_env
    c = _ctx_with_env(RMX_TUNE_DEAL_XCD=0)
    yield c
    c.close()


@pytest.mark.parametrize("n", [16, 19, 37, 64])
def test_every_sample_is_processed_under_its_own_row(ctx, ctx_batch_order, n):
    rng = np.random.default_rng(400 + n)
    H, W = 48, 64
    img = rng.integers(0, 256, (n, H, W, 3), dtype=np.uint8)
    roi = np.empty((n, 4), np.uint32)
    for i in range(n):
        w, h = int(rng.integers(8, W + 1)), int(rng.integers(8, H + 1))
        roi[i] = (int(rng.integers(0, W - w + 1)), int(rng.integers(0, H - h + 1)), w, h)
    mirror = rng.integers(0, 2, n).astype(np.uint32)
    scale = rng.uniform(0.5, 2.0, 3 * n).astype(np.float32)  # per-sample constants: a mixed-up sample cannot pass
    bias = rng.uniform(-1.0, 1.0, 3 * n).astype(np.float32)
    dw = (rng.integers(1, 8, n) * 8).astype(np.uint32)
    dh = rng.integers(4, 40, n).astype(np.uint32)
    OH, OW = int(dh.max()), int(dw.max())
    src = _gpu(img)
    sd = ops.desc(n, H, W, ops.NHWC, ops.UINT8)

    # bilinear resize + normalise (the streaming kernel: 192-byte rows), triangular, crop-mirror-normalise, warp
    exp_lin = orc.resize(img, roi, dw, dh, OH, OW, interp=orc.LINEAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NCHW, dtype=ops.FP16,
                         flags=orc.F_QUANTIZE_U8)
    exp_tri = orc.resize(img, roi, dw, dh, OH, OW, interp=orc.TRIANGULAR, mirror=mirror, scale=scale, bias=bias, layout=ops.NHWC, dtype=ops.FP32)
    crop = roi.copy()
    exp_cmn = orc.crop_mirror_normalize(img, crop, scale, bias, mirror, H, W, ops.NCHW, ops.FP32)
    angle = rng.uniform(-40, 40, n).astype(np.float32)
    m = np.stack([orc.rotate_matrix(a) for a in angle])
    full = np.tile(np.array([0, 0, W, H], np.uint32), (n, 1))
    wdw, wdh = np.full(n, W, np.uint32), np.full(n, H, np.uint32)
    exp_rot = orc.warp_affine(img, full, m, wdw, wdh, H, W, interp=orc.LINEAR)
    outs = {}
    for c in (ctx, ctx_batch_order):
        op = ops.Resize(c, sd, ops.desc(n, OH, OW, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
        op.update_cmn(roi, dw, dh, scale, bias, mirror)
        o1 = op.alloc_output(); op.launch(src, o1)
        op2 = ops.Resize(c, sd, ops.desc(n, OH, OW, ops.NHWC, ops.FP32), ops.TRIANGULAR)
        op2.update_cmn(roi, dw, dh, scale, bias, mirror)
        o2 = op2.alloc_output(); op2.launch(src, o2)
        op3 = ops.CropMirrorNormalize(c, sd, ops.desc(n, H, W, ops.NCHW, ops.FP32))
        op3.update(crop, scale, bias, mirror)
        o3 = op3.alloc_output(); op3.launch(src, o3)
        op4 = ops.Rotate(c, sd, sd, ops.LINEAR)
        op4.update(full, angle, wdw, wdh)
        o4 = op4.alloc_output(); op4.launch(src, o4)
        c.sync()
        outs[c] = [o.cpu().numpy() for o in (o1, o2, o3, o4)]
    for got in outs.values():
        for i in range(n):
            assert np.array_equal(got[0][i, :, :dh[i], :dw[i]].view(np.uint16), exp_lin[i, :, :dh[i], :dw[i]].view(np.uint16)), "bilinear, sample %d" % i
            assert np.array_equal(got[1][i, :dh[i], :dw[i]].view(np.uint32), exp_tri[i, :dh[i], :dw[i]].view(np.uint32)), "triangular, sample %d" % i
            ch, cw = int(crop[i, 3]), int(crop[i, 2])
            assert np.array_equal(got[2][i, :, :ch, :cw].view(np.uint32), exp_cmn[i, :, :ch, :cw].view(np.uint32)), "crop-mirror-normalise, sample %d" % i
            assert np.array_equal(got[3][i], exp_rot[i]), "rotate, sample %d" % i
