"""The C++ host layer (rocal_amd/host: rocAL's Node / Graph / Parameter interface and rocal* entry points)
driving the HIP kernels through the C ABI, checked against the oracle. Each scenario is a small
pipeline built with the reference's own API calls; the expected result is computed here from the
oracle's restatement of the parameter laws and of the pixel arithmetic."""
import os
import subprocess

import numpy as np
import pytest

from oracle import orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_CHECK = os.path.join(ROOT, "rocal_amd", "lib", "host_check")
SEED = 77  # set by the driver with rocalSetSeed
N, H, W = 6, 80, 96
ROIS = [(96, 80), (70, 60), (96, 64), (81, 80), (50, 77), (33, 41)]  # (w, h)
MEAN, STD = [123.675, 116.28, 103.53], [58.395, 57.12, 57.375]


def _image():
    rng = np.random.default_rng(5)
    base = rng.integers(0, 256, (N, H // 4 + 1, W // 4 + 1, 3)).astype(np.float32)
    img = np.repeat(np.repeat(base, 4, axis=1), 4, axis=2)[:, :H, :W]
    img += rng.normal(0, 12, img.shape)
    return np.clip(np.rint(img), 0, 255).astype(np.uint8)


def _run(scenario, tmp_path, n_out, shapes):
    img = _image()
    img.tofile(tmp_path / "input.bin")
    with open(tmp_path / "meta.txt", "w") as f:
        f.write("%d %d %d\n" % (N, H, W))
        for w, h in ROIS:
            f.write("%d %d\n" % (w, h))
    print("host_check pipeline", scenario, flush=True)
    p = subprocess.run([HOST_CHECK, "pipeline", scenario, str(tmp_path)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, (p.returncode, p.stdout, p.stderr)
    outs = []
    for b in range(2):
        row = []
        for k in range(n_out):
            dt, shape = shapes[k]
            row.append((np.fromfile(tmp_path / ("out%d_b%d.bin" % (k, b)), dtype=dt).reshape(shape),
                        np.loadtxt(tmp_path / ("roi%d_b%d.txt" % (k, b)), dtype=np.int64).reshape(N, 4)))
        outs.append(row)
    return img, outs, p.stdout


def _roi():
    return np.array([[0, 0, w, h] for w, h in ROIS], np.uint32)


def _coin_batches(batches):
    """The driver's first parameter: CustomRand<int>({0,1},{.5,.5}) seeded with the first value of the
    seed sequence; one draw in its constructor, then N draws per batch."""
    g = orc.MT19937(int(orc.seed_seq_generate([SEED], 1024)[0]))
    g.custom_index([0.5, 0.5])
    return [np.array([g.custom_index([0.5, 0.5]) for _ in range(N)], np.uint32) for _ in range(batches)]


def _same(got, exp, what):
    assert got.shape == exp.shape, what
    assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), "%s: %d values differ" % (what, (got != exp).sum())


def test_crop_mirror_normalize_node(tmp_path):
    img, outs, _ = _run("cmn", tmp_path, 1, [(np.float32, (N, 3, 40, 48))])
    crop = np.stack([orc.fixed_crop(w, h, 48, 40, anchor=(0.5, 0.5)) for w, h in ROIS])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    mirrors = _coin_batches(2)
    assert mirrors[0].tolist() != mirrors[1].tolist() or mirrors[0].any()
    for b in range(2):
        got, roi = outs[b][0]
        exp = orc.crop_mirror_normalize(img, crop, scale, bias, mirrors[b], 40, 48, orc.NCHW, orc.FP32)
        _same(got, exp, "cmn batch %d" % b)
        assert np.array_equal(roi[:, 2:], crop[:, 2:])  # the output ROI is the crop size


def test_random_resized_crop_then_cmn_runs_as_one_kernel(tmp_path):
    img, outs, log = _run("rrc_cmn", tmp_path, 1, [(np.float16, (N, 3, 56, 56))])
    assert "intermediate_elided 1" in log  # the u8 tensor between the two nodes is never materialised
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.5), s(1.2), s(0.3), s(0.7), w, h) for w, h in ROIS])
    full = np.full(N, 64, np.uint32)
    mid = orc.resize(img, window, full, full, 64, 64, interp=orc.LINEAR)  # the u8 image of the two-node graph
    # CropResizeNode publishes the crop size (capped to 64) as the ROI of its output; the CMN crop follows it
    mid_w, mid_h = np.minimum(window[:, 2], 64), np.minimum(window[:, 3], 64)
    crop = np.stack([orc.fixed_crop(int(w), int(h), 56, 56, anchor=(0.5, 0.5)) for w, h in zip(mid_w, mid_h)])
    assert (crop[:, 2] < 56).any() and (crop[:, 2] == 56).any()
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    mirrors = _coin_batches(2)
    for b in range(2):
        got, roi = outs[b][0]
        exp = orc.crop_mirror_normalize(mid, crop, scale, bias, mirrors[b], 56, 56, orc.NCHW, orc.FP16)
        _same(got, exp, "rrc+cmn batch %d" % b)
        assert np.array_equal(roi[:, 2:], crop[:, 2:])


@pytest.mark.parametrize("scenario", ["rrc_twist_cmn", "rrc_contrast_cmn", "rrc_exposure_cmn"])
def test_random_resized_crop_colour_cmn_runs_as_one_kernel(tmp_path, scenario):
    img, outs, log = _run(scenario, tmp_path, 1, [(np.float16, (N, 3, 56, 56))])
    assert "intermediate_elided 1" in log and "second_intermediate_elided 1" in log  # neither u8 tensor is materialised
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.5), s(1.2), s(0.3), s(0.7), w, h) for w, h in ROIS])
    full = np.full(N, 64, np.uint32)
    mid = orc.resize(img, window, full, full, 64, 64, interp=orc.LINEAR)
    mid_w, mid_h = np.minimum(window[:, 2], 64), np.minimum(window[:, 3], 64)
    one = lambda v: np.full(N, v, np.float32)
    # the colour node works on the ROI the resize node publishes for its output
    mid_roi = np.stack([np.zeros(N), np.zeros(N), mid_w, mid_h], -1).astype(np.uint32)
    if scenario == "rrc_twist_cmn":
        mid = orc.color_twist(mid, mid_roi, one(1.2), one(8.0), one(40.0), one(1.3))
    elif scenario == "rrc_contrast_cmn":
        mid = orc.contrast(mid, mid_roi, one(1.4), one(100.0))
    else:
        mid = orc.exposure(mid, mid_roi, one(0.4))
    crop = np.stack([orc.fixed_crop(int(w), int(h), 56, 56, anchor=(0.5, 0.5)) for w, h in zip(mid_w, mid_h)])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    mirrors = _coin_batches(2)
    for b in range(2):
        got, roi = outs[b][0]
        exp = orc.crop_mirror_normalize(mid, crop, scale, bias, mirrors[b], 56, 56, orc.NCHW, orc.FP16)
        _same(got, exp, "%s batch %d" % (scenario, b))
        assert np.array_equal(roi[:, 2:], crop[:, 2:])


@pytest.mark.parametrize("edge", ["textbook", "device"])
def test_caller_built_against_the_public_header_alone(tmp_path, edge):
    """tests/cpp/api_caller.cpp sees include/rocal_api_mi355x.h and nothing else of this repository: CropResize -> ColorTwist ->
    CropMirrorNormalize, two batches, read as a program written for rocAL reads them (rocalGetOutputTensors(ctx)->at(0)->copy_data,
    dims, strides, copy_roi, rocalCopyToOutput), the second with the output bound to memory the caller allocated (set_mem_handle);
    the timers of rocalGetTimingInfo. Same expected values as the three reference nodes run one after the other, under both
    rules for the right / lower neighbour at a window's edge (ROCAL_BILINEAR_EDGE: the textbook clamp, and the last-but-one
    pixel of the reference's device kernel, rocal_hip_kernels.cpp:339-345)."""
    img = _image()
    img.tofile(tmp_path / "input.bin")
    with open(tmp_path / "meta.txt", "w") as f:
        f.write("%d %d %d\n" % (N, H, W))
        for w, h in ROIS:
            f.write("%d %d\n" % (w, h))
    exe = os.path.join(ROOT, "rocal_amd", "lib", "api_caller")
    print("api_caller", edge, flush=True)
    env = dict(os.environ)
    env.pop("ROCAL_BILINEAR_EDGE", None)
    if edge == "device":
        env["ROCAL_BILINEAR_EDGE"] = "device"
    p = subprocess.run([exe, str(tmp_path)], capture_output=True, text=True, timeout=110, env=env)
    assert p.returncode == 0, (p.returncode, p.stdout, p.stderr)
    assert "intermediates_elided 1" in p.stdout and p.stdout.strip().endswith("ok")
    t = dict(zip(*[iter(p.stdout.split("timing_us ")[1].split("\n")[0].split())] * 2))
    assert int(t["process"]) > 0 and int(t["update"]) > 0 and int(t["load"]) == 0 and int(t["transfer"]) > 0  # (transfer: rocalCopyToOutput)
    assert "timing_after_reset 0" in p.stdout
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.5), s(1.2), s(0.3), s(0.7), w, h) for w, h in ROIS])
    full = np.full(N, 64, np.uint32)
    mid = orc.resize(img, window, full, full, 64, 64, interp=orc.LINEAR, flags=orc.F_BILINEAR_EDGE_QUIRK if edge == "device" else 0)
    if edge == "device":  # the two rules differ on this input (else the second run would prove nothing)
        assert not np.array_equal(mid, orc.resize(img, window, full, full, 64, 64, interp=orc.LINEAR))
    mid_w, mid_h = np.minimum(window[:, 2], 64), np.minimum(window[:, 3], 64)
    one = lambda v: np.full(N, v, np.float32)
    mid_roi = np.stack([np.zeros(N), np.zeros(N), mid_w, mid_h], -1).astype(np.uint32)
    mid = orc.color_twist(mid, mid_roi, one(1.2), one(8.0), one(40.0), one(1.3))
    crop = np.stack([orc.fixed_crop(int(w), int(h), 56, 56, anchor=(0.5, 0.5)) for w, h in zip(mid_w, mid_h)])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    mirrors = _coin_batches(2)
    for b in range(2):
        got = np.fromfile(tmp_path / ("out_b%d.bin" % b), dtype=np.float16).reshape(N, 3, 56, 56)
        _same(got, orc.crop_mirror_normalize(mid, crop, scale, bias, mirrors[b], 56, 56, orc.NCHW, orc.FP16), "caller batch %d" % b)
        roi = np.loadtxt(tmp_path / ("roi_b%d.txt" % b), dtype=np.int64).reshape(N, 4)
        assert np.array_equal(roi[:, 2:], crop[:, 2:])


def test_resize_colortwist_flip_chain_with_intermediate_tensors(tmp_path):
    img, outs, _ = _run("chain", tmp_path, 2, [(np.uint8, (N, 32, 40, 3))] * 2)
    dw, dh = np.full(N, 40, np.uint32), np.full(N, 32, np.uint32)
    a = orc.resize(img, _roi(), dw, dh, 32, 40, interp=orc.LINEAR)
    roi_a = np.array([[0, 0, 40, 32]] * N, np.uint32)
    one = lambda v: np.full(N, v, np.float32)
    b_exp = orc.color_twist(a, roi_a, one(1.1), one(5.0), one(30.0), one(1.2))
    c_exp = orc.crop_mirror_normalize(b_exp, roi_a, None, None, np.ones(N, np.uint32), 32, 40, orc.NHWC, orc.UINT8, vflip=np.zeros(N, np.uint32))
    for b in range(2):
        _same(outs[b][0][0], b_exp, "colour twist of the resized image")
        _same(outs[b][1][0], c_exp, "flip of the twisted image")
        assert np.array_equal(outs[b][1][1], roi_a)  # same-size nodes share the ROI of their input


def test_rotate_node(tmp_path):
    img, outs, _ = _run("rotate", tmp_path, 1, [(np.uint8, (N, H, W, 3))])
    m = np.stack([orc.rotate_matrix(30.0)] * N)
    exp = orc.warp_affine(img, _roi(), m, np.full(N, W, np.uint32), np.full(N, H, np.uint32), H, W, interp=orc.LINEAR)
    _same(outs[1][0][0], exp, "rotate")


def test_warp_affine_node(tmp_path):
    img, outs, _ = _run("warp", tmp_path, 1, [(np.uint8, (N, 48, 56, 3))])
    # rocAL's fill order x0,y0,x1,y1,o0,o1 (node_warp_affine.cpp:43-48)
    m = np.stack([orc.affine_from_rocal([1.05, -0.08, 0.1, 0.95, 3.0, -2.0])] * N)
    exp = orc.warp_affine(img, _roi(), m, np.full(N, 56, np.uint32), np.full(N, 48, np.uint32), 48, 56, interp=orc.LINEAR)
    _same(outs[0][0][0], exp, "warp affine")


def test_resize_mirror_normalize_node_with_shorter_side_policy(tmp_path):
    img, outs, _ = _run("rmn", tmp_path, 1, [(np.float16, (N, 3, 96, 96))])
    sizes = np.array([orc.resize_out_size(w, h, 48, 48, 2, 96, 96) for w, h in ROIS], np.uint32)
    sizes = np.minimum(sizes, 96)
    assert len({tuple(s) for s in sizes.tolist()}) > 3  # ragged destination sizes
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    exp = orc.resize(img, _roi(), sizes[:, 0], sizes[:, 1], 96, 96, interp=orc.LINEAR, mirror=np.ones(N, np.uint32), scale=scale, bias=bias,
                     layout=orc.NCHW, dtype=orc.FP16)
    for b in range(2):
        got, roi = outs[b][0]
        _same(got, exp, "resize-mirror-normalize")
        assert np.array_equal(roi[:, 2:], sizes)


def test_crop_variants_and_point_ops(tmp_path):
    img, outs, _ = _run("crops", tmp_path, 5, [(np.uint8, (N, 24, 32, 3)), (np.uint8, (N, 20, 30, 3)), (np.uint8, (N, 28, 36, 3)),
                                                 (np.uint8, (N, H, W, 3)), (np.uint8, (N, H, W, 3))])
    o = outs[1]
    centre = np.stack([orc.fixed_crop(w, h, 32, 24, anchor=(0.5, 0.5)) for w, h in ROIS])
    _same(o[0][0], orc.crop_mirror_normalize(img, centre, None, None, None, 24, 32, orc.NHWC, orc.UINT8), "centre crop")
    placed = np.stack([orc.fixed_crop(w, h, 30, 20, x1=5, y1=7) for w, h in ROIS])
    _same(o[1][0], orc.crop_mirror_normalize(img, placed, None, None, None, 20, 30, orc.NHWC, orc.UINT8), "placed crop")
    window = np.stack([orc.fixed_crop(w, h, 50, 40) for w, h in ROIS])
    exp = orc.resize(img, window, np.full(N, 36, np.uint32), np.full(N, 28, np.uint32), 28, 36, interp=orc.LINEAR, mirror=np.ones(N, np.uint32))
    _same(o[2][0], exp, "resize-crop-mirror")
    one = lambda v: np.full(N, v, np.float32)
    _same(o[3][0], orc.brightness(img, _roi(), one(1.2), one(10.0)), "brightness")
    _same(o[4][0], orc.contrast(img, _roi(), one(1.3), one(70.0)), "contrast")


def test_gamma_exposure_colour_temperature_blend_nodes(tmp_path):
    full = (np.uint8, (N, H, W, 3))
    img, outs, _ = _run("points", tmp_path, 5, [full] * 5)
    one = lambda v: np.full(N, v, np.float32)
    for o in outs:  # fixed parameters: both batches give the same result
        _same(o[0][0], orc.gamma(img, _roi(), one(2.2)), "gamma")
        _same(o[1][0], orc.exposure(img, _roi(), one(0.6)), "exposure")
        _same(o[2][0], orc.color_temperature(img, _roi(), np.full(N, 40, np.int32)), "colour temperature")
        bright = orc.brightness(img, _roi(), one(0.5), one(100.0))
        _same(o[3][0], bright, "brightness")
        _same(o[4][0], orc.blend(img, bright, _roi(), one(0.3)), "blend of the source and a node's output")


def test_tensor_read_as_a_second_input_is_not_fused_away(tmp_path):
    """resize -> {CropMirrorNormalize, Blend(other, resized)}: the resized tensor has two readers, one of them through a
    node's second input, so the pair resize -> CropMirrorNormalize stays two launches and the tensor exists."""
    img, outs, stdout = _run("second_reader", tmp_path, 3, [(np.float32, (N, 3, 32, 40)), (np.uint8, (N, 32, 40, 3)), (np.uint8, (N, 32, 40, 3))])
    assert "intermediate_elided 0" in stdout
    dw, dh = np.full(N, 40, np.uint32), np.full(N, 32, np.uint32)
    mid = orc.resize(img, _roi(), dw, dh, 32, 40, interp=orc.LINEAR)
    other = orc.resize(img, _roi(), dw, dh, 32, 40, interp=orc.NEAREST)
    whole = np.tile(np.array([0, 0, 40, 32], np.uint32), (N, 1))
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    for o in outs:
        _same(o[0][0], orc.crop_mirror_normalize(mid, whole, scale, bias, np.zeros(N, np.uint32), 32, 40, orc.NCHW, orc.FP32), "CropMirrorNormalize of the resized tensor")
        _same(o[1][0], other, "nearest resize")
        _same(o[2][0], orc.blend(other, mid, whole, np.full(N, 0.25, np.float32)), "blend with the resized tensor as second input")


def test_normalize_and_transpose_nodes(tmp_path):
    """rocalNormalize (computed per-channel statistics; given statistics with scale and shift) and rocalTranspose ({1,0,2} and
    {2,0,1}) on the ragged source: values from the oracle / numpy, output ROIs swapped where the permutation swaps."""
    img, outs, _ = _run("normalize_transpose", tmp_path, 4, [(np.float32, (N, H, W, 3)), (np.float16, (N, H, W, 3)), (np.uint8, (N, W, H, 3)),
                                                             (np.uint8, (N, 3, H, W))])
    e0 = orc.normalize(img, _roi(), axis_mask=3, layout=orc.NHWC, dtype=orc.FP32)
    e1 = orc.normalize(img, _roi(), axis_mask=7, mean=[10.0, 20.0, 30.0], stddev=[2.0, 4.0, 8.0], scale=3.0, shift=1.0, layout=orc.NHWC, dtype=orc.FP16)
    for o in outs:
        for i, (w, h) in enumerate(ROIS):
            _same(o[0][0][i, :h, :w], e0[i, :h, :w], "normalize, computed statistics, sample %d" % i)
            _same(o[1][0][i, :h, :w], e1[i, :h, :w], "normalize, given statistics, sample %d" % i)
            _same(o[2][0][i, :w, :h], np.ascontiguousarray(img[i, :h, :w].transpose(1, 0, 2)), "transpose {1,0,2}, sample %d" % i)
            _same(o[3][0][i, :, :h, :w], np.ascontiguousarray(img[i, :h, :w].transpose(2, 0, 1)), "transpose {2,0,1}, sample %d" % i)
        assert np.array_equal(o[2][1][:, 2:], np.array([[h, w] for w, h in ROIS]))  # width and height swapped
        assert np.array_equal(o[3][1][:, 2:], np.array([[w, h] for w, h in ROIS]))


def test_to_tensor_of_the_u8_output(tmp_path):
    """rocalToTensor (rocal_api_data_transfer.cpp:30-52 -> MasterGraph::to_tensor): planar fp16 with reversed
    channels of the whole output, then an interleaved fp32 tensor of its top-left max_roi corner."""
    img, outs, _ = _run("to_tensor", tmp_path, 1, [(np.uint8, (N, 32, 40, 3))])
    dw, dh = np.full(N, 40, np.uint32), np.full(N, 32, np.uint32)
    a = orc.resize(img, _roi(), dw, dh, 32, 40, interp=orc.LINEAR)
    _same(outs[1][0][0], a, "resized u8 output")
    f32 = lambda *v: np.array(v, np.float32)
    t0 = np.fromfile(tmp_path / "tt0.bin", dtype=np.float16).reshape(N, 3, 32, 40)
    _same(t0, orc.to_tensor(a, f32(1 / f32(58.395)[0], 1 / f32(57.12)[0], 1 / f32(57.375)[0]), f32(-2.0, -1.5, -1.0), reverse_channels=True,
                            layout=orc.NCHW, dtype=orc.FP16), "planar fp16 tensor")
    t1 = np.fromfile(tmp_path / "tt1.bin", dtype=np.float32).reshape(N, 24, 32, 3)
    _same(t1, orc.to_tensor(np.ascontiguousarray(a[:, :24, :32]), f32(0.5, 0.25, 2.0), f32(1.0, 0.0, -3.0), layout=orc.NHWC, dtype=orc.FP32),
          "interleaved fp32 tensor of the 24x32 corner")


def test_api_errors_follow_the_reference(tmp_path):
    _image().tofile(tmp_path / "input.bin")
    with open(tmp_path / "meta.txt", "w") as f:
        f.write("%d %d %d\n" % (N, H, W) + "".join("%d %d\n" % r for r in ROIS))
    p = subprocess.run([HOST_CHECK, "pipeline", "errors", str(tmp_path)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0 and "errors_bad_mask 0" in p.stdout, (p.returncode, p.stdout, p.stderr[-2000:])


# ---------------------------------------------------------------- bounding boxes through the metadata nodes

def _boxes():
    """Per sample: a list of (l, t, r, b) inside the sample's ROI and a list of labels; one sample has no box."""
    rng = np.random.default_rng(8)
    boxes, labels = [], []
    for i, (w, h) in enumerate(ROIS):
        k = 0 if i == 3 else int(rng.integers(1, 5))
        bs = []
        for _ in range(k):
            l, t = rng.uniform(0, w * 0.7), rng.uniform(0, h * 0.7)
            bs.append((np.float32(l), np.float32(t), np.float32(min(w, l + rng.uniform(4, w * 0.6))), np.float32(min(h, t + rng.uniform(4, h * 0.6)))))
        boxes.append(bs)
        labels.append([int(x) for x in rng.integers(1, 90, k)])
    return boxes, labels


def _run_meta(scenario, tmp_path):
    from oracle import meta  # noqa: F401  (imported here so that a missing file fails this test only)
    boxes, labels = _boxes()
    with open(tmp_path / "boxes.txt", "w") as f:
        for bs, ls in zip(boxes, labels):
            f.write("%d\n" % len(bs))
            for b, l in zip(bs, ls):
                f.write("%.9g %.9g %.9g %.9g %d\n" % (b[0], b[1], b[2], b[3], l))
    img = _image()
    img.tofile(tmp_path / "input.bin")
    with open(tmp_path / "meta.txt", "w") as f:
        f.write("%d %d %d\n" % (N, H, W))
        for w, h in ROIS:
            f.write("%d %d\n" % (w, h))
    print("host_check pipeline", scenario, flush=True)
    p = subprocess.run([HOST_CHECK, "pipeline", scenario, str(tmp_path)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, (p.returncode, p.stdout, p.stderr)
    got = []
    for b in range(2):
        tok = open(tmp_path / ("boxes_b%d.txt" % b)).read().split()
        k, batch = 0, []
        for _ in range(N):
            c = int(tok[k]); k += 1
            bs, ls = [], []
            for _ in range(c):
                bs.append(tuple(np.float32(float(v)) for v in tok[k:k + 4]))
                ls.append(int(tok[k + 4]))
                k += 5
            batch.append((bs, ls))
        got.append(batch)
    return boxes, labels, got


def _same_boxes(got, exp, what, rtol=0.0):
    gb, gl = got
    eb, el = exp
    assert len(gb) == len(eb), (what, gb, eb)
    assert gl[:len(el)] == el and all(v == 0 for v in gl[len(el):]), (what, gl, el)
    for g, e in zip(gb, eb):
        if rtol:
            assert np.allclose(np.array(g, np.float32), np.array(e, np.float32), rtol=rtol, atol=1e-4), (what, g, e)
        else:
            assert np.array_equal(np.array(g, np.float32).view(np.uint32), np.array(e, np.float32).view(np.uint32)), (what, g, e)


def test_boxes_through_crop_mirror_normalize(tmp_path):
    from oracle import meta
    boxes, labels, got = _run_meta("meta_cmn", tmp_path)
    crop = np.stack([orc.fixed_crop(w, h, 48, 40, anchor=(0.5, 0.5)) for w, h in ROIS])
    mirrors = _coin_batches(2)
    for b in range(2):
        for i in range(N):
            x1, y1, cw, ch = (int(v) for v in crop[i])
            _same_boxes(got[b][i], meta.crop_mirror_normalize(boxes[i], labels[i], x1, y1, cw, ch, int(mirrors[b][i])), "cmn boxes, batch %d sample %d" % (b, i))


def test_boxes_through_resize_then_flip(tmp_path):
    from oracle import meta
    boxes, labels, got = _run_meta("meta_resize_flip", tmp_path)
    for i, (w, h) in enumerate(ROIS):
        rb, rl = meta.resize(boxes[i], labels[i], w, h, 40, 32)
        _same_boxes(got[1][i], meta.flip(rb, rl, 40, 32, 1, 1), "resize+flip boxes, sample %d" % i)


def test_boxes_through_rotate(tmp_path):
    """cos and sin come from the C library on one side and from Python's on the other: compared to 1e-5."""
    from oracle import meta
    boxes, labels, got = _run_meta("meta_rotate", tmp_path)
    for i, (w, h) in enumerate(ROIS):
        _same_boxes(got[0][i], meta.rotate(boxes[i], labels[i], w, h, W, H, 30.0), "rotate boxes, sample %d" % i, rtol=1e-5)


def test_boxes_through_resize_crop_mirror(tmp_path):
    from oracle import meta
    boxes, labels, got = _run_meta("meta_rcm", tmp_path)
    window = np.stack([orc.fixed_crop(w, h, 50, 40) for w, h in ROIS])
    for i in range(N):
        x1, y1, cw, ch = (int(v) for v in window[i])
        _same_boxes(got[1][i], meta.resize_crop_mirror(boxes[i], labels[i], x1, y1, x1 + cw, y1 + ch, 36, 28, 1), "rcm boxes, sample %d" % i)


def test_boxes_through_crop_then_resize_mirror_normalize(tmp_path):
    from oracle import meta
    boxes, labels, got = _run_meta("meta_crop_then_rmn", tmp_path)
    placed = np.stack([orc.fixed_crop(w, h, 30, 20, x1=5, y1=7) for w, h in ROIS])
    for i in range(N):
        x1, y1, cw, ch = (int(v) for v in placed[i])
        cb, cl = meta.crop(boxes[i], labels[i], x1, y1, cw, ch)
        _same_boxes(got[0][i], meta.resize_mirror_normalize(cb, cl, cw, ch, 60, 40, 1), "crop+rmn boxes, sample %d" % i)


def test_boxes_through_crop_resize(tmp_path):
    from oracle import meta
    boxes, labels, got = _run_meta("meta_crop_resize", tmp_path)
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.5), s(1.2), s(0.3), s(0.7), w, h) for w, h in ROIS])
    for i in range(N):
        x1, y1, cw, ch = (int(v) for v in window[i])
        _same_boxes(got[1][i], meta.crop_resize(boxes[i], labels[i], x1, y1, x1 + cw, y1 + ch, 64, 64), "crop-resize boxes, sample %d" % i)
