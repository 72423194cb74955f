"""Host layer (rocal_amd/host, C++) against the oracle's restatement of rocAL's parameter laws.

The C++ side uses the real std::mt19937 / std::seed_seq of libstdc++, the oracle its own hand-written
generators: agreement here also pins the oracle's generators against the C++ standard library."""
import json
import os
import subprocess

import numpy as np
import pytest

from oracle import orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_CHECK = os.path.join(ROOT, "rocal_amd", "lib", "host_check")
SEED = 42
ROIS = [(640, 480), (240, 240), (333, 500), (500, 333), (64, 48), (1000, 200)]


@pytest.fixture(scope="module")
def host():
    if not os.path.exists(HOST_CHECK):
        pytest.fail("rocal_amd/lib/host_check is not built (run __graft_entry__.build())")
    out = subprocess.run([HOST_CHECK, "params", str(SEED)], check=True, capture_output=True, text=True, timeout=60).stdout
    return json.loads(out)


@pytest.fixture(scope="module")
def seeds():
    return orc.seed_seq_generate([SEED], 1024)


def test_seed_sequence_matches_libstdcxx(host, seeds):
    assert host["seeds"] == [int(s) for s in seeds[:4]]


def test_uniform_float_law(host, seeds):
    g = orc.MT19937(int(seeds[4]))
    exp = [g.uniform_f32(0.08, 1.0) for _ in range(13)]  # constructor draw + 12 renewals
    assert np.array_equal(np.float32(host["uniform_f"]), np.float32(exp))


def test_uniform_int_law_truncates(host, seeds):
    g = orc.MT19937(int(seeds[5]))
    exp = [g.uniform_i32(0, 1) for _ in range(13)]
    assert host["uniform_i"] == exp
    # truncation of u in [0,1]: 1 only when the raw draw is the generator's maximum
    assert set(exp) == {0}


def test_custom_rand_law(host, seeds):
    g = orc.MT19937(int(seeds[6]))
    vals = [10, 20, 30, 40]
    exp = [vals[g.custom_index([0.1, 0.4, 0.3, 0.2])] for _ in range(13)]
    assert host["custom_i"] == exp
    assert len(set(exp)) >= 3


def test_default_node_parameter_uses_factory_seed_and_renews_per_sample(host):
    g = orc.MT19937(SEED)
    g.uniform_i32(0, 1)  # constructor
    exp = [g.uniform_i32(0, 1) for _ in range(3 * 8)]
    assert host["mirror_default"] == exp


def _uniform(seeds, k, lo, hi):
    return orc.FParam.uniform(lo, hi, int(seeds[k]))


def test_random_resized_crop_windows(host, seeds):
    area, aspect = _uniform(seeds, 7, 0.08, 1.0), _uniform(seeds, 8, 0.75, 1.333)
    xd, yd = _uniform(seeds, 9, 0.0, 1.0), _uniform(seeds, 10, 0.0, 1.0)
    exp = []
    for _ in range(3):
        for p in (area, aspect, xd, yd):  # the per-batch renewal of every registered parameter
            p.renew()
        for w, h in ROIS:
            exp += [int(v) for v in orc.random_crop(area, aspect, xd, yd, w, h)]
    assert host["rrc_windows"] == exp
    win = np.array(exp).reshape(-1, 4)
    rois = np.array(ROIS * 3)
    assert (win[:, 0] + win[:, 2] <= rois[:, 0]).all() and (win[:, 1] + win[:, 3] <= rois[:, 1]).all()
    assert (win[:, 2] > 0).all() and (win[:, 3] > 0).all()


def test_factor_crop_windows(host, seeds):
    hf, wf = _uniform(seeds, 15, 0.55, 0.95), _uniform(seeds, 16, 0.55, 0.95)
    xd, yd = _uniform(seeds, 17, 0.01, 0.99), _uniform(seeds, 18, 0.01, 0.99)
    exp = []
    for _ in range(2):
        for p in (hf, wf, xd, yd):
            p.renew()
        for w, h in ROIS:
            exp += [int(v) for v in orc.factor_crop(hf, wf, xd, yd, w, h)]
    assert host["factor_windows"] == exp


def test_anchored_crop_windows(host):
    exp = []
    for w, h in ROIS:
        exp += [int(v) for v in orc.fixed_crop(w, h, 224, 200, anchor=(0.5, 0.5))]
    assert host["fixed_windows"] == exp


def test_resize_size_policy(host):
    cases = [(640, 480, 256, 0, 0), (640, 480, 0, 256, 0), (640, 480, 300, 200, 1), (640, 480, 256, 256, 2), (480, 640, 256, 256, 2),
             (640, 480, 256, 256, 3), (333, 500, 0, 300, 3), (333, 500, 300, 0, 2), (1000, 200, 256, 256, 2)]
    exp = []
    for sw, sh, dw, dh, mode in cases:
        for mw, mh in ((0, 0), (400, 300)):
            exp += list(orc.resize_out_size(sw, sh, dw, dh, mode, mw, mh))
    assert host["resize_sizes"] == exp


def test_oracle_crop_laws_known_answers():
    """Arithmetic done by hand, so that the oracle's crop laws are pinned by more than the host code."""
    s = orc.FParam.simple
    # area .5 of 100x100 at aspect 1: w = h = trunc(sqrt(5000)) = 70; drift .5 of the slack 30 -> 15
    assert list(orc.random_crop(s(0.5), s(1.0), s(0.5), s(0.5), 100, 100)) == [15, 15, 70, 70]
    # aspect 4/3 (exactly representable products): target 0.48*100*100 = 4800; w = trunc(sqrt(6400)) = 80, h = trunc(sqrt(3600)) = 60
    w = orc.random_crop(s(0.48), s(4 / 3), s(0.0), s(1.0), 100, 100)
    assert list(w[2:]) in ([80, 60], [79, 59], [80, 59], [79, 60])  # fp32 rounding of 0.48 and 4/3 may fall either side
    assert w[0] == 0 and w[1] == 100 - w[3]
    # no candidate can fit (area 1 => w == W is not strictly smaller): centre crop; 300x100 has ratio 3 > 1.333 -> h=100, w=trunc(133.3)=133
    assert list(orc.random_crop(s(1.0), s(1.0), s(0.5), s(0.5), 300, 100)) == [(300 - 133) // 2, 0, 133, 100]
    # ratio 1/3 < 0.75 -> w=100, h=trunc(100/0.75)=133
    assert list(orc.random_crop(s(1.0), s(1.0), s(0.5), s(0.5), 100, 300)) == [0, (300 - 133) // 2, 100, 133]
    # factor crop: trunc(.5*101)=50, trunc(.25*80)=20; drifts trunc(.5*51)=25, trunc(.99*60)=59
    assert list(orc.factor_crop(s(0.25), s(0.5), s(0.5), s(0.99), 101, 80)) == [25, 59, 50, 20]


# ---------------------------------------------------------------- metadata laws: the restatement against hand-computed cases

def test_box_laws_known_answers():
    from oracle import meta
    f = np.float32
    boxes, labels = [(10, 10, 50, 40), (0, 0, 5, 5), (28, 20, 60, 60)], [3, 4, 5]
    # crop window (5,7)+(30x20): box 0 keeps 425/1200 of its area (kept, clipped, shifted); box 1 is outside;
    # box 2 keeps 7*7/1280 (dropped)
    assert meta.crop(boxes, labels, 5, 7, 30, 20) == ([(f(5), f(3), f(30), f(20))], [3])
    # nothing left -> the whole crop with label 0
    assert meta.crop([(0, 0, 5, 5)], [9], 50, 50, 10, 8) == ([(f(0), f(0), f(10), f(8))], [0])
    # mirror inside the crop: l' = w - r, r' = w - l
    assert meta.crop_mirror_normalize(boxes[:1], labels[:1], 5, 7, 30, 20, 1) == ([(f(0), f(3), f(25), f(20))], [3])
    # crop + resize by exactly 2 in x and 3 in y
    assert meta.crop_resize(boxes[:1], labels[:1], 5, 7, 35, 27, 60, 60) == ([(f(10), f(9), f(60), f(60))], [3])
    # resize-crop-mirror: mirror in the crop frame, then scale
    assert meta.resize_crop_mirror(boxes[:1], labels[:1], 5, 7, 35, 27, 60, 60, 1) == ([(f(0), f(9), f(50), f(60))], [3])
    # plain resize doubles; an empty sample gets one zero box and no label
    assert meta.resize([(1, 2, 3, 4)], [7], 10, 10, 20, 20) == ([(f(2), f(4), f(6), f(8))], [7])
    assert meta.resize([], [], 10, 10, 20, 20) == ([(f(0), f(0), f(0), f(0))], [])
    # resize-mirror-normalize mirrors with the "- 1" of the reference
    assert meta.resize_mirror_normalize([(1, 2, 3, 4)], [7], 10, 10, 20, 20, 1) == ([(f(13), f(4), f(17), f(8))], [7])
    # flipping twice is the identity
    once = meta.flip([(1, 2, 3, 4)], [7], 10, 8, 1, 1)
    assert once == ([(f(7), f(4), f(9), f(6))], [7]) and meta.flip(*once, 10, 8, 1, 1) == ([(f(1), f(2), f(3), f(4))], [7])
    # rotation by 0 degrees about equal centres keeps the box (its left/top are min(0, .) first, then clipped to the image)
    assert meta.rotate([(10, 10, 50, 40)], [3], 96, 80, 96, 80, 0.0) == ([(f(0), f(0), f(50), f(40))], [3])
    # overlap measure: intersection over the first box's area, or over the union
    assert meta.overlap((0, 0, 10, 10), (5, 5, 15, 15)) == 0.25
    assert abs(meta.overlap((0, 0, 10, 10), (5, 5, 15, 15), True) - 25.0 / 175.0) < 1e-7


# ---- decoder-side random-resized-crop law (RocalRandomCropDecParam) ----
# The C++ class draws with libstdc++'s distributions. The expectation below restates those algorithms from their published
# definitions over the oracle's generator: generate_canonical<float,24> on a 32-bit engine (one draw, divided by 2^32 in
# float arithmetic, 1.0 replaced by the float below it) and uniform_int_distribution<int> on a 32-bit engine (Lemire's
# multiply-shift with rejection). libm supplies logf / expf / sqrtf / roundf, as it does for the C++ class.

def _libm():
    import ctypes as C
    m = C.CDLL("libm.so.6")
    for f in ("logf", "expf", "sqrtf", "roundf"):
        getattr(m, f).restype = C.c_float
        getattr(m, f).argtypes = [C.c_float]
    return m


class _StdDraws:
    def __init__(self, seed):
        self.g = orc.MT19937(int(seed) & 0xFFFFFFFF)
        self.draws = 0

    def raw(self):
        self.draws += 1
        return self.g.next()

    def canonical(self):
        r = np.float32(self.raw()) / np.float32(4294967296.0)
        return np.nextafter(np.float32(1), np.float32(0)) if r >= np.float32(1) else r

    def real(self, a, b):
        a, b = np.float32(a), np.float32(b)
        return np.float32(np.float32(self.canonical() * np.float32(b - a)) + a)

    def integer(self, lo, hi):
        rng_ = hi - lo + 1
        prod = self.raw() * rng_
        low = prod & 0xFFFFFFFF
        if low < rng_:
            thresh = ((1 << 32) - rng_) % rng_
            while low < thresh:
                prod = self.raw() * rng_
                low = prod & 0xFFFFFFFF
        return lo + (prod >> 32)


def _dec_window(seed, H, W, area=(0.08, 1.0), ratio=(3.0 / 4.0, 4.0 / 3.0), attempts=10):
    m, f32 = _libm(), np.float32
    d = _StdDraws(seed)
    lo_r, hi_r = f32(ratio[0]), f32(ratio[1])
    log_lo, log_hi = f32(m.logf(lo_r)), f32(m.logf(hi_r))
    a_lo, a_hi = f32(area[0]), f32(area[1])
    max_hw = f32(1) / lo_r
    min_area = f32(W * H) * a_lo
    max_w = max(1, int(f32(H) * hi_r))
    max_h = max(1, int(f32(W) * max_hw))
    if f32(H * max_w) < min_area:
        h, w = H, max_w
    elif f32(W * max_h) < min_area:
        h, w = max_h, W
    else:
        for _ in range(attempts):
            scale = d.real(a_lo, a_hi)
            target = f32(scale * f32(H * W))
            r = f32(m.expf(d.real(log_lo, log_hi)))
            w = max(1, int(m.roundf(m.sqrtf(f32(target * r)))))
            h = max(1, int(m.roundf(m.sqrtf(f32(target / r)))))
            rr = f32(w) / f32(h)
            if w <= W and h <= H and lo_r <= rr <= hi_r:
                break
        else:
            max_area = f32(f32(a_hi * f32(W)) * f32(H))
            rr = f32(W) / f32(H)
            if rr > hi_r:
                h, w = H, max_w
            elif rr < lo_r:
                h, w = max_h, W
            else:
                h, w = H, W
            s = min(f32(1), max_area / f32(w * h))
            rs = f32(m.sqrtf(s))
            w = max(1, int(f32(w) * rs))
            h = max(1, int(f32(h) * rs))
    x = d.integer(0, W - w)
    y = d.integer(0, H - h)
    return (x, y, w, h), d.draws


def _host_windows(seed, shapes, **kw):
    from rocal_amd import workloads as wl
    return wl.random_crop_dec_windows(seed, [s[0] for s in shapes], [s[1] for s in shapes], **kw)


def test_decoder_crop_windows_follow_the_reference_law():
    rng = np.random.default_rng(8)
    shapes = [(int(rng.integers(240, 641)), int(rng.integers(240, 641))) for _ in range(256)]
    shapes += [(1, 1), (2, 3), (3, 2), (5, 5), (7, 1), (1, 9), (16, 4000), (4000, 16)]
    seeds = orc.seed_seq_generate([1235], len(shapes))
    got = _host_windows(1235, shapes)
    retried = 0
    for i, (H, W) in enumerate(shapes):
        exp, draws = _dec_window(seeds[i], H, W)
        assert tuple(int(v) for v in got[i]) == exp, "sample %d (%dx%d)" % (i, H, W)
        retried += draws > 4
    assert retried >= 20  # the retry branch is exercised (about a fifth of ImageNet-like shapes need a second attempt)
    x, y, w, h = got[:, 0].astype(int), got[:, 1].astype(int), got[:, 2].astype(int), got[:, 3].astype(int)
    Hs, Ws = np.array([s[0] for s in shapes]), np.array([s[1] for s in shapes])
    assert np.all(w >= 1) and np.all(h >= 1) and np.all(x + w <= Ws) and np.all(y + h <= Hs)


def test_decoder_crop_windows_hand_computed_cases():
    # Too wide (H=10, W=1000): max width = int(10 * 4/3) = 13; 10*13 = 130 < 0.08*10000 = 800 -> 10 x 13 without any
    # attempt; y has a single possible value. Too tall is the transpose: max height = int(10 / 0.75) = 13.
    got = _host_windows(7, [(10, 1000), (1000, 10)])
    assert got[0, 2:].tolist() == [13, 10] and got[0, 1] == 0 and 0 <= got[0, 0] <= 987
    assert got[1, 2:].tolist() == [10, 13] and got[1, 0] == 0 and 0 <= got[1, 1] <= 987
    # A degenerate law (area exactly 1, ratio exactly 1) on a square image: sqrt(H*W) = H, the whole image, at (0, 0).
    got = _host_windows(7, [(64, 64), (300, 300)], area=(1.0, 1.0), ratio=(1.0, 1.0))
    assert got.tolist() == [[0, 0, 64, 64], [0, 0, 300, 300]]
    # The same law on a 2:1 image can never satisfy h <= H: after ten attempts the fallback takes the side limits
    # (ratio 2 > 1 -> H x int(H*1)), area scale min(1, W*H / (H*H)) = 1 -> a centred-law square of side H, x uniform.
    got = _host_windows(7, [(100, 200)], area=(1.0, 1.0), ratio=(1.0, 1.0))
    assert got[0, 2:].tolist() == [100, 100] and got[0, 1] == 0 and 0 <= got[0, 0] <= 100
    # Fallback with shrink: area at most 0.25 of a 2:1 image, ratio exactly 1, attempts 0 -> H x H scaled by
    # sqrt(0.25*200*100 / (100*100)) = sqrt(0.5): width int(100*0.70710677) = 70, then height int(100*0.70710677) = 70.
    got = _host_windows(7, [(100, 200)], area=(0.25, 0.25), ratio=(1.0, 1.0), attempts=0)
    assert got[0, 2:].tolist() == [70, 70]


def test_decoder_crop_windows_statistics():
    # Large sample on one shape: the area fraction is uniform on [0.08, 1] conditioned on fitting, the position uniform.
    n = 4000
    got = _host_windows(99, [(480, 640)] * n).astype(np.float64)
    frac = got[:, 2] * got[:, 3] / (480 * 640)
    ratio = got[:, 2] / got[:, 3]
    assert 0.079 <= frac.min() and frac.max() <= 1.0
    assert np.all(ratio >= 0.75 - 1e-6) and np.all(ratio <= 4 / 3 + 1e-6)
    assert abs(np.mean(np.log(ratio))) < 0.05      # log-uniform about 1 (fit conditioning leaves a small tilt)
    free = 640 - got[:, 2]
    assert abs(np.mean(got[free > 50, 0] / free[free > 50]) - 0.5) < 0.03


def test_loader_ring_shutdown_protocol():
    """The ring of packed batches in host memory (no HIP call on this path): a loader thread blocked on the full ring is woken
    by stop() / release() / unblock_writer() and leaves with an exception, never with a slot that is still full; release() frees
    the slots only after the thread has left; a consumer blocked on the empty ring is woken the same way; reset() reopens
    the ring (rocAL/source/loaders/image/image_loader.cpp:84,126-127,241; circular_buffer.cpp:299-343)."""
    exe = os.path.join(ROOT, "rocal_amd", "lib", "host_check")
    p = subprocess.run([exe, "ring"], capture_output=True, text=True, timeout=60)
    assert p.returncode == 0, (p.stdout, p.stderr)
    lines = p.stdout.strip().splitlines()
    assert lines[-1] == "ring ok" and all(l.endswith(" ok") for l in lines)
    for name in ("stop_wakes_loader", "release_wakes_loader", "unblock_without_room_is_an_error", "release_wakes_reader",
                 "reader_turned_away_after_stop", "ring_usable_after_reset", "oldest_batch_intact", "writer_continues_after_pop"):
        assert name + " ok" in lines
