"""A pipeline written with the Python fn.* layer on the GPU: resize_crop -> color_twist -> crop_mirror_normalize with the
output bound to a torch tensor the caller owns (the node writes straight into it: what the reference does with a copy after
the run), and a warp / flip pipeline read through its own buffers. Expected values from the oracle."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import fn, types
from rocal_amd.pipeline import Pipeline

pytestmark = pytest.mark.gpu

N, H, W = 6, 80, 96
ROIS = [(96, 80), (70, 60), (96, 64), (81, 80), (50, 77), (33, 41)]  # (w, h)
MEAN, STD = [123.675, 116.28, 103.53], [58.395, 57.12, 57.375]


def _image():
    rng = np.random.default_rng(15)
    return rng.integers(0, 256, (N, H, W, 3), dtype=np.uint8)


def test_random_resized_crop_colour_twist_cmn_into_a_torch_tensor():
    import torch
    img = _image()
    pipe = Pipeline(batch_size=N, device_id=0, seed=77)
    with pipe:
        src = pipe.device_source(W, H)
        a = fn.resize_crop(src, resize_width=64, resize_height=64, crop_area_factor=0.5, crop_aspect_ratio=1.2, x_drift=0.3, y_drift=0.7)
        c = fn.color_twist(a, brightness=1.2, contrast=8.0, hue=40.0, saturation=1.3)
        out = fn.crop_mirror_normalize(c, crop=(56, 56), mean=MEAN, std=STD, mirror=1, output_layout=types.NCHW, output_dtype=types.FLOAT16)
        pipe.set_outputs(out)
    mine = torch.zeros((N, 3, 56, 56), dtype=torch.float16, device="cuda")
    pipe.bind_output(out, mine)
    pipe.build()
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.5), s(1.2), s(0.3), s(0.7), w, h) for w, h in ROIS])
    full = np.full(N, 64, np.uint32)
    mid = orc.resize(img, window, full, full, 64, 64, interp=orc.LINEAR)
    mid_w, mid_h = np.minimum(window[:, 2], 64), np.minimum(window[:, 3], 64)
    one = lambda v: np.full(N, v, np.float32)
    mid_roi = np.stack([np.zeros(N), np.zeros(N), mid_w, mid_h], -1).astype(np.uint32)
    mid = orc.color_twist(mid, mid_roi, one(1.2), one(8.0), one(40.0), one(1.3))
    crop = np.stack([orc.fixed_crop(int(w), int(h), 56, 56, anchor=(0.5, 0.5)) for w, h in zip(mid_w, mid_h)])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    exp = orc.crop_mirror_normalize(mid, crop, scale, bias, np.ones(N, np.uint32), 56, 56, orc.NCHW, orc.FP16)
    dimg = torch.from_numpy(img).cuda()
    for batch in range(2):
        mine.zero_()
        pipe.feed(src, dimg, [w for w, _ in ROIS], [h for _, h in ROIS])
        pipe.rocal_run()
        pipe.get_output_tensors()  # the consumer's wait for the batch
        got = mine.cpu().numpy()
        assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), "batch %d: %d values differ" % (batch, int((got != exp).sum()))
        assert np.array_equal(np.array(pipe.output_roi(out))[:, 2:], crop[:, 2:])
    t = pipe.timing_info()
    assert t["process_time"] > 0 and t["parameter_update_time"] > 0 and t["load_time"] == 0
    pipe.release()


def test_warp_affine_and_flip_pipeline():
    import torch
    img = _image()
    pipe = Pipeline(batch_size=N, device_id=0, seed=3)
    with pipe:
        src = pipe.device_source(W, H)
        wa = fn.warp_affine(src, dest_width=56, dest_height=48, matrix=[1.05, 0.1, -0.08, 0.95, 3.0, -2.0])
        fl = fn.flip(wa, horizontal=1, vertical=0)
        pipe.set_outputs(wa, fl)
    t_wa = torch.zeros((N, 48, 56, 3), dtype=torch.uint8, device="cuda")
    t_fl = torch.zeros((N, 48, 56, 3), dtype=torch.uint8, device="cuda")
    pipe.bind_output(wa, t_wa)  # both outputs land in the caller's tensors; the flip node reads the first one from there
    pipe.bind_output(fl, t_fl)
    pipe.build()
    # (sizes as uint32 arrays: handed to the library without a per-element conversion)
    pipe.feed(src, torch.from_numpy(img).cuda(), np.array([w for w, _ in ROIS], np.uint32), np.array([h for _, h in ROIS], np.uint32))
    pipe.rocal_run()
    pipe.get_output_tensors()  # the consumer's wait for the batch
    # matrix [x0, x1, y0, y1, o0, o1] reaches the node as rocAL's fill order x0, y0, x1, y1, o0, o1 (node_warp_affine.cpp:43-48)
    m = np.stack([orc.affine_from_rocal([1.05, -0.08, 0.1, 0.95, 3.0, -2.0])] * N)
    roi = np.array([[0, 0, w, h] for w, h in ROIS], np.uint32)
    exp = orc.warp_affine(img, roi, m, np.full(N, 56, np.uint32), np.full(N, 48, np.uint32), 48, 56, interp=orc.LINEAR)
    assert np.array_equal(t_wa.cpu().numpy(), exp)
    assert np.array_equal(t_fl.cpu().numpy(), exp[:, :, ::-1])
    pipe.release()


def test_output_through_dlpack():
    """The output tensor handed to torch as a DLPack capsule: the torch tensor aliases the buffer the node wrote (same device
    address, no copy) and holds the oracle's values."""
    import torch
    img = _image()
    pipe = Pipeline(batch_size=N, device_id=0, seed=3)
    with pipe:
        src = pipe.device_source(W, H)
        out = fn.crop_mirror_normalize(src, crop=(32, 40), mean=MEAN, std=STD, mirror=1, output_layout=types.NCHW, output_dtype=types.FLOAT)
        pipe.set_outputs(out)
    pipe.build()
    dimg = torch.from_numpy(img).cuda()
    pipe.feed(src, dimg, [w for w, _ in ROIS], [h for _, h in ROIS])
    pipe.rocal_run()
    pipe.get_output_tensors()  # the consumer's wait for the batch
    t = torch.from_dlpack(pipe.output_dlpack(out))
    assert t.is_cuda and t.dtype == torch.float32 and tuple(t.shape) == (N, 3, 32, 40)
    from rocal_amd import backend
    assert t.data_ptr() == backend.Backend().tensorBuffer(out)
    crop = np.stack([orc.fixed_crop(w, h, 40, 32, anchor=(0.5, 0.5)) for w, h in ROIS])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    exp = orc.crop_mirror_normalize(img, crop, scale, bias, np.ones(N, np.uint32), 32, 40, orc.NCHW, orc.FP32)
    got = t.cpu().numpy()
    for i in range(N):
        cw, ch = int(crop[i, 2]), int(crop[i, 3])
        assert np.array_equal(got[i, :, :ch, :cw], exp[i, :, :ch, :cw]), "sample %d" % i
    del t
    pipe.release()
