"""Packed source batches through the host layer: images of different sizes are placed one by one into the pinned slot of a ring
(PackedCircularBuffer, standing where the reference's loader pads every image into a [N, Hmax, Wmax, 3] batch), pushed, copied
once, and read by the first node of the graph through the ragged-source layout. Results against the oracle on the padded batch."""
import numpy as np
import pytest

from oracle import orc
from rocal_amd import fn, types
from rocal_amd.pipeline import Pipeline

pytestmark = pytest.mark.gpu

N, HMAX, WMAX = 6, 80, 96
MEAN, STD = [123.675, 116.28, 103.53], [58.395, 57.12, 57.375]


def _batch(seed):
    rng = np.random.default_rng(seed)
    sizes = [(int(rng.integers(20, WMAX + 1)), int(rng.integers(20, HMAX + 1))) for _ in range(N)]  # (w, h)
    sizes[0] = (WMAX, HMAX)
    sizes[1] = (63, 31)  # 189-byte rows: 3 bytes of padding per row
    images = [rng.integers(0, 256, (h, w, 3), dtype=np.uint8) for w, h in sizes]
    padded = np.zeros((N, HMAX, WMAX, 3), np.uint8)
    for i, im in enumerate(images):
        padded[i, :im.shape[0], :im.shape[1]] = im
    return sizes, images, padded


def _expect(padded, sizes):
    s = orc.FParam.simple
    window = np.stack([orc.random_crop(s(0.6), s(1.1), s(0.25), s(0.75), w, h) for w, h in sizes])
    full = np.full(N, 48, np.uint32)
    mid = orc.resize(padded, window, full, full, 48, 48, interp=orc.LINEAR)
    mid_w, mid_h = np.minimum(window[:, 2], 48), np.minimum(window[:, 3], 48)
    crop = np.stack([orc.fixed_crop(int(w), int(h), 40, 40, anchor=(0.5, 0.5)) for w, h in zip(mid_w, mid_h)])
    scale, bias = orc.cmn_scale_bias(MEAN, STD, N)
    return orc.crop_mirror_normalize(mid, crop, scale, bias, np.zeros(N, np.uint32), 40, 40, orc.NCHW, orc.FP16)


def test_packed_batches_through_the_ring():
    import torch
    pipe = Pipeline(batch_size=N, device_id=0, seed=5)
    with pipe:
        src = pipe.packed_source(WMAX, HMAX, queue_depth=3)
        a = fn.resize_crop(src, resize_width=48, resize_height=48, crop_area_factor=0.6, crop_aspect_ratio=1.1, x_drift=0.25, y_drift=0.75)
        out = fn.crop_mirror_normalize(a, crop=(40, 40), mean=MEAN, std=STD, mirror=0, output_layout=types.NCHW, output_dtype=types.FLOAT16)
        pipe.set_outputs(out)
    mine = torch.zeros((N, 3, 40, 40), dtype=torch.float16, device="cuda")
    pipe.bind_output(out, mine)
    pipe.build()
    with pytest.raises(RuntimeError, match="no batch"):
        pipe.rocal_run()  # nothing pushed yet
    batches = [_batch(100 + k) for k in range(5)]
    # two batches ahead of the consumer (a ring of three holds two finished batches), images placed in any order
    for k in (0, 1):
        for i in reversed(range(N)):
            pipe.place_image(src, i, batches[k][1][i])
        pipe.push(src)
    assert pipe.queued_batches(src) == 2
    for k in range(5):
        mine.zero_()
        torch.cuda.synchronize()  # (the pipeline's stream is not ordered against torch's)
        pipe.rocal_run()
        pipe.get_output_tensors()  # the consumer's wait for the batch
        got = mine.cpu().numpy()
        exp = _expect(batches[k][2], batches[k][0])
        assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), "batch %d: %d values differ" % (k, int((got != exp).sum()))
        if k + 2 < 5:  # the slot just read is free again: the ring goes round
            for i in range(N):
                pipe.place_image(src, i, batches[k + 2][1][i])
            pipe.push(src)
    assert pipe.queued_batches(src) == 0
    pipe.release()


def test_packed_source_errors():
    pipe = Pipeline(batch_size=2, device_id=0, seed=5)
    with pipe:
        src = pipe.packed_source(32, 32, queue_depth=2, slot_bytes=32 * 32 * 3 + 300)
        out = fn.flip(src, horizontal=1)
        pipe.set_outputs(out)
    pipe.build()
    img = np.zeros((32, 32, 3), np.uint8)
    pipe.place_image(src, 0, img)
    with pytest.raises(RuntimeError, match="twice"):
        pipe.place_image(src, 0, img)
    with pytest.raises(RuntimeError, match="exceeds its slot"):
        pipe.place_image(src, 1, img)           # the slot holds one full image and a bit
    with pytest.raises(RuntimeError, match="exceeds the source"):
        pipe.place_image(src, 1, np.zeros((33, 8, 3), np.uint8))
    with pytest.raises(RuntimeError, match="not placed"):
        pipe.push(src)
    pipe.place_image(src, 1, np.zeros((3, 8, 3), np.uint8))
    pipe.push(src)
    pipe.rocal_run()
    pipe.get_output_tensors()  # the consumer's wait for the batch
    pipe.release()


def test_loader_thread_and_consumer():
    """A loader thread assembles and pushes eight batches through a ring of two slots (it blocks while the ring is full), the
    main thread waits for a batch, runs and checks it."""
    import threading
    import torch
    pipe = Pipeline(batch_size=N, device_id=0, seed=5)
    with pipe:
        src = pipe.packed_source(WMAX, HMAX, queue_depth=2)
        a = fn.resize_crop(src, resize_width=48, resize_height=48, crop_area_factor=0.6, crop_aspect_ratio=1.1, x_drift=0.25, y_drift=0.75)
        out = fn.crop_mirror_normalize(a, crop=(40, 40), mean=MEAN, std=STD, mirror=0, output_layout=types.NCHW, output_dtype=types.FLOAT16)
        pipe.set_outputs(out)
    mine = torch.zeros((N, 3, 40, 40), dtype=torch.float16, device="cuda")
    pipe.bind_output(out, mine)
    pipe.build()
    batches = [_batch(200 + k) for k in range(8)]
    failed = []

    def loader():
        try:
            for k in range(8):
                for i in range(N):
                    pipe.place_image(src, i, batches[k][1][i])
                pipe.push(src)
        except Exception as e:  # noqa: BLE001
            failed.append(e)

    th = threading.Thread(target=loader)
    th.start()
    try:
        for k in range(8):
            pipe.wait_for_batch(src)
            mine.zero_()  # the nodes write the valid region of every sample only
            torch.cuda.synchronize()
            pipe.rocal_run()
            pipe.get_output_tensors()  # the consumer's wait for the batch
            got = mine.cpu().numpy()
            exp = _expect(batches[k][2], batches[k][0])
            assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), "batch %d" % k
        th.join(timeout=30)
        assert not th.is_alive() and not failed
    finally:
        pipe.release()  # (wakes the loader if a check above failed while it was blocked on the full ring)
        th.join(timeout=30)


def test_release_wakes_a_loader_blocked_on_the_full_ring():
    """The shut-down protocol of the reference's loaders (image_loader.cpp:84,126-127: unblock_writer / unblock_reader before the
    buffer goes): a loader thread, not a daemon, blocked in place_image on a full ring; release() from the main thread; the
    thread leaves within a second with the error recorded, and never with a slot that was still full."""
    import threading
    import time
    pipe = Pipeline(batch_size=N, device_id=0, seed=5)
    with pipe:
        src = pipe.packed_source(WMAX, HMAX, queue_depth=2)
        out = fn.crop_mirror_normalize(src, crop=(40, 40), mean=MEAN, std=STD, mirror=0, output_layout=types.NCHW, output_dtype=types.FLOAT16)
        pipe.set_outputs(out)
    pipe.build()
    _, images, _ = _batch(7)
    state = {"pushed": 0, "error": None}

    def loader():
        try:
            for _ in range(4):  # the ring holds one finished batch: the second batch's first image blocks
                for i in range(N):
                    pipe.place_image(src, i, images[i])
                pipe.push(src)
                state["pushed"] += 1
        except Exception as e:  # noqa: BLE001
            state["error"] = e

    th = threading.Thread(target=loader)
    th.start()
    deadline = time.time() + 10
    while state["pushed"] < 1 and time.time() < deadline:
        time.sleep(0.01)
    time.sleep(0.2)
    assert th.is_alive() and state["pushed"] == 1 and state["error"] is None  # blocked on the full ring
    t0 = time.time()
    pipe.release()
    th.join(timeout=5)
    assert not th.is_alive() and time.time() - t0 < 1.0
    assert state["pushed"] == 1 and "released" in str(state["error"])
