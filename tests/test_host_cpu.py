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
