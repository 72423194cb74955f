"""CPU tests that pin the parts of the oracle which closed forms at integer coordinates leave open:
the fractional path of the warp (weight order, neighbour choice, far-edge clamp, the out-of-ROI rule),
nearest-neighbour resize, and the reciprocal form of the colour twist's divisions. Every expected value
is computed here in integers, in float64, or by a library routine - never by retyping the oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import orc

RNG = np.random.default_rng(77001)


def _img(n, h, w, rng=RNG):
    return rng.integers(0, 256, (n, h, w, 3), dtype=np.uint8)


def _full(n, h, w):
    return np.tile(np.array([0, 0, w, h], np.uint32), (n, 1))


def _rne_div(num, den):
    """round-half-to-even of num/den for non-negative integer arrays"""
    q, r = np.divmod(num, den)
    up = (2 * r > den) | ((2 * r == den) & (q % 2 == 1))
    return q + up


# ------------------------------------------------------------------ warp: fractional translations, exact dyadic blends

@pytest.mark.parametrize("tx,ty", [(0.5, 0.25), (0.25, 0.5), (0.75, 0.0), (0.0, 0.75)])
def test_warp_fractional_translation_is_exact_dyadic_blend(tx, ty):
    # source = destination + (tx, ty) with 0 <= tx,ty < 1: floor = the destination pixel, weights (tx, ty).
    # Different x and y fractions: swapping wx and wy, or taking the wrong neighbour, changes the integers below.
    h, w = 13, 17
    img = _img(1, h, w)
    m = np.array([[1, 0, tx, 0, 1, ty]], np.float32)
    out = orc.warp_affine(img, _full(1, h, w), m, [w], [h], h, w)
    a = img[0].astype(np.int64)
    right = np.concatenate([a[:, 1:], a[:, -1:]], axis=1)  # neighbour beyond the last column repeats it
    down = np.concatenate([a[1:], a[-1:]], axis=0)
    downright = np.concatenate([right[1:], right[-1:]], axis=0)
    fx, fy = int(tx * 4), int(ty * 4)  # quarters
    num = a * (4 - fy) * (4 - fx) + right * (4 - fy) * fx + down * fy * (4 - fx) + downright * fy * fx
    exp = _rne_div(num, 16)
    assert np.array_equal(out[0].astype(np.int64), exp)


def test_warp_negative_fraction_takes_left_upper_neighbours_and_zeroes_the_first_row_and_column():
    # source = destination - (0.5, 0.25): floor is one pixel up/left, weights (0.5, 0.75); floor == -1 is outside the ROI
    h, w = 9, 11
    img = _img(1, h, w)
    m = np.array([[1, 0, -0.5, 0, 1, -0.25]], np.float32)
    out = orc.warp_affine(img, _full(1, h, w), m, [w], [h], h, w)
    a = img[0].astype(np.int64)
    tl, tr, bl, br = a[:-1, :-1], a[:-1, 1:], a[1:, :-1], a[1:, 1:]
    exp = _rne_div(tl * 1 * 2 + tr * 1 * 2 + bl * 3 * 2 + br * 3 * 2, 16)  # (1-wy)=1/4, wy=3/4, wx=1/2
    assert np.array_equal(out[0, 1:, 1:].astype(np.int64), exp)
    assert not out[0, 0].any() and not out[0, :, 0].any()


def test_warp_out_of_roi_rule_at_the_window_edges():
    # ROI strictly inside the image, filled with 200; everything around it is 50. A pure x translation moves the
    # source coordinate across both edges of the window.
    h, w = 8, 24
    img = np.full((1, h, w, 3), 50, np.uint8)
    x0, y0, rw, rh = 5, 2, 10, 4
    img[0, y0:y0 + rh, x0:x0 + rw] = 200
    roi = np.array([[x0, y0, rw, rh]], np.uint32)
    for t, expect in [
        (0.0, lambda x: 200),                       # identity: every pixel inside
        (0.5, lambda x: 200),                       # floor(sx) = x0+x <= xhi; at x = rw-1 the right neighbour is clamped to xhi (not 50)
        (1.0, lambda x: 200 if x <= rw - 2 else 0),   # floor(sx) = x0+x+1: x = rw-1 lands on xhi+1 -> outside -> 0
        (-0.25, lambda x: 200 if x >= 1 else 0),    # floor(sx) = x0+x-1: x = 0 lands on x0-1 -> outside -> 0 (not a blend with 50)
        (-1.0, lambda x: 200 if x >= 1 else 0),
    ]:
        m = np.array([[1, 0, t, 0, 1, 0]], np.float32)
        out = orc.warp_affine(img, roi, m, [rw], [rh], rh, rw)
        for x in range(rw):
            assert (out[0, :, x] == expect(x)).all(), (t, x, out[0, 0, x])
    # same along y, with the far-row clamp
    for t, expect in [(0.5, lambda y: 200), (1.0, lambda y: 200 if y <= rh - 2 else 0), (-0.5, lambda y: 200 if y >= 1 else 0)]:
        m = np.array([[1, 0, 0, 0, 1, t]], np.float32)
        out = orc.warp_affine(img, roi, m, [rw], [rh], rh, rw)
        for y in range(rh):
            assert (out[0, y] == expect(y)).all(), (t, y)


def _warp_f64(img, roi, m, dw, dh):
    """float64 evaluation of the stated law: centres w>>1, destination -> source, bilinear, 0 outside the ROI,
    far neighbours clamped. Returns (value, distance of the source point to the nearest integer grid line, inside-the-ROI mask)."""
    x0, y0, w, h = [int(v) for v in roi]
    xhi, yhi = x0 + w - 1, y0 + h - 1
    out = np.zeros((dh, dw, 3), np.float64)
    margin = np.full((dh, dw), 1.0)
    inside = np.zeros((dh, dw), bool)
    for y in range(dh):
        for x in range(dw):
            xr, yr = x - (dw >> 1), y - (dh >> 1)
            sx = xr * float(m[0]) + yr * float(m[1]) + float(m[2]) + (x0 + (w >> 1))
            sy = xr * float(m[3]) + yr * float(m[4]) + float(m[5]) + (y0 + (h >> 1))
            fx, fy = math.floor(sx), math.floor(sy)
            margin[y, x] = min(sx - fx, fx + 1 - sx, sy - fy, fy + 1 - sy)
            if fx < x0 or fy < y0 or fx > xhi or fy > yhi:
                continue
            inside[y, x] = True
            wx, wy = sx - fx, sy - fy
            ix1, iy1 = min(fx + 1, xhi), min(fy + 1, yhi)
            p = img.astype(np.float64)
            out[y, x] = (p[fy, fx] * (1 - wy) * (1 - wx) + p[fy, ix1] * (1 - wy) * wx + p[iy1, fx] * wy * (1 - wx) + p[iy1, ix1] * wy * wx)
    return out, margin, inside


@pytest.mark.parametrize("seed", range(6))
def test_warp_brute_force_float64_rotation_scale_shift(seed):
    rng = np.random.default_rng(500 + seed)
    h, w = 12, 14
    img = _img(1, h, w, rng)
    x0, y0, rw, rh = 2, 1, 9, 9  # ROI off the origin: the source centre is x0 + (w>>1)
    dw, dh = 13, 10              # destination of another size: its centre is dw>>1
    th = math.radians(rng.uniform(-40, 40))
    s = rng.uniform(0.7, 1.3)
    m = np.array([math.cos(th) * s, -math.sin(th) * s, rng.uniform(-1.5, 1.5),
                  math.sin(th) * s, math.cos(th) * s, rng.uniform(-1.5, 1.5)], np.float32)
    out = orc.warp_affine(img, np.array([[x0, y0, rw, rh]], np.uint32), m[None], [dw], [dh], dh, dw)
    exp, margin, inside = _warp_f64(img[0], (x0, y0, rw, rh), m, dw, dh)
    # where the source point is not within 1e-4 of a grid line, fp32 and float64 agree on floor() and on the ROI test
    safe = margin > 1e-4
    assert safe.mean() > 0.9
    assert inside[safe].sum() > 10 and (~inside)[safe].sum() > 10  # both branches are exercised
    assert not out[0][safe & ~inside].any()
    diff = np.abs(out[0].astype(np.float64) - np.clip(np.rint(exp), 0, 255))
    assert diff[safe].max() <= 1
    # and the fp32 value before rounding is within 1e-3 of the float64 one: a 1-LSB step only at a rounding boundary
    near_half = np.abs(exp - np.floor(exp) - 0.5) < 1e-3
    assert (diff[safe][~near_half[safe]] == 0).all()


def test_warp_interior_matches_torch_grid_sample():
    rng = np.random.default_rng(9)
    h = w = 40
    img = _img(1, h, w, rng)
    th = math.radians(17.0)
    m = np.array([math.cos(th) * 1.1, -math.sin(th) * 1.1, 0.37, math.sin(th) * 1.1, math.cos(th) * 1.1, -0.81], np.float32)
    out = orc.warp_affine(img, _full(1, h, w), m[None], [w], [h], h, w)
    ys, xs = np.meshgrid(np.arange(h), np.arange(w), indexing="ij")
    xr, yr = xs - (w >> 1), ys - (h >> 1)
    sx = xr * float(m[0]) + yr * float(m[1]) + float(m[2]) + (w >> 1)
    sy = xr * float(m[3]) + yr * float(m[4]) + float(m[5]) + (h >> 1)
    grid = torch.from_numpy(np.stack([2 * sx / (w - 1) - 1, 2 * sy / (h - 1) - 1], axis=-1)[None]).double()
    t = torch.from_numpy(img.transpose(0, 3, 1, 2).astype(np.float64))
    ref = torch.nn.functional.grid_sample(t, grid, mode="bilinear", padding_mode="zeros", align_corners=True)[0].permute(1, 2, 0).numpy()
    interior = (sx >= 0) & (sx <= w - 1.001) & (sy >= 0) & (sy <= h - 1.001)  # all four taps inside the image
    assert interior.sum() > 600
    d = np.abs(out[0].astype(np.float64) - ref)
    assert d[interior].max() <= 0.5 + 1e-3  # the rounded value is the nearest integer of torch's
    outside = (np.floor(sx) < 0) | (np.floor(sx) > w - 1) | (np.floor(sy) < 0) | (np.floor(sy) > h - 1)
    assert outside.sum() > 50 and not out[0][outside].any()


def test_warp_nearest_picks_the_rounded_source_pixel():
    h, w = 9, 10
    img = _img(1, h, w)
    m = np.array([[1, 0, 0.4, 0, 1, 0.6]], np.float32)  # rounds to (x, y+1)
    out = orc.warp_affine(img, _full(1, h, w), m, [w], [h], h, w, interp=orc.NEAREST)
    assert np.array_equal(out[0, :-1], img[0, 1:])
    assert not out[0, -1].any()  # row h is outside


# ------------------------------------------------------------------ nearest-neighbour resize: expected indices written by hand

def _resize_nearest(img, dw, dh):
    n, h, w, _ = img.shape
    return orc.resize(img, _full(n, h, w), [dw] * n, [dh] * n, dh, dw, interp=orc.NEAREST, layout=orc.NHWC, dtype=orc.UINT8)


def test_nearest_scale_one_is_identity():
    img = _img(2, 7, 9)
    assert np.array_equal(_resize_nearest(img, 9, 7), img)


def test_nearest_integer_downscale_picks_a_stated_pixel():
    img = _img(1, 12, 18)
    # 2x: the source coordinate of output d is 2d + 0.5, equally far from 2d and 2d+1: the tie goes to 2d+1
    assert np.array_equal(_resize_nearest(img, 9, 6), img[:, 1::2, 1::2])
    # 3x: the source coordinate is 3d + 1 exactly: the middle pixel of each triple
    assert np.array_equal(_resize_nearest(img, 6, 4), img[:, 1::3, 1::3])


def test_nearest_upscale_replicates():
    img = _img(1, 5, 6)
    assert np.array_equal(_resize_nearest(img, 12, 10), img.repeat(2, axis=1).repeat(2, axis=2))
    assert np.array_equal(_resize_nearest(img, 18, 15), img.repeat(3, axis=1).repeat(3, axis=2))


def test_nearest_respects_the_roi_and_mirror():
    img = _img(1, 10, 12)
    roi = np.array([[3, 2, 6, 4]], np.uint32)
    out = orc.resize(img, roi, [6], [4], 4, 6, interp=orc.NEAREST, mirror=[1], layout=orc.NHWC, dtype=orc.UINT8)
    assert np.array_equal(out[0], img[0, 2:6, 3:9][:, ::-1])


# ------------------------------------------------------------------ colour twist: every RGB triple, reciprocals against true divisions

def _twist_division_form(rgb, alpha, beta, hue_deg, sat):
    """The HSV round trip with true divisions (delta/cmax, num/delta), numpy fp32, no reciprocal table and no fused
    multiply-add. rgb: [P,3] uint8. Returns the unrounded fp32 result [P,3]."""
    f = np.float32
    r, g, b = (rgb[:, k].astype(f) for k in range(3))
    cmax = np.maximum(np.maximum(r, g), b)
    cmin = np.minimum(np.minimum(r, g), b)
    delta = cmax - cmin
    nz = delta != 0
    safe_d = np.where(nz, delta, f(1))
    safe_m = np.where(cmax != 0, cmax, f(1))
    s = np.where(nz, delta / safe_m, f(0)).astype(f)
    is_r = cmax == r
    is_g = ~is_r & (cmax == g)
    num = np.where(is_r, g - b, np.where(is_g, b - r, r - g)).astype(f)
    add = np.where(is_r, f(0), np.where(is_g, f(2), f(4))).astype(f)
    shift = f(math.fmod(hue_deg, 360.0))
    if shift < 0:
        shift = f(shift + f(360))
    shift = f(shift / f(60))
    hh = np.where(nz, num / safe_d + add, f(0)).astype(f) + shift
    hh = np.where(hh < 0, hh + f(6), hh)
    hh = np.where(hh >= 6, hh - f(6), hh).astype(f)
    s = np.clip(s * f(sat), f(0), f(1)).astype(f)
    hi = np.floor(hh).astype(np.int32)
    hf = (hh - hi.astype(f)).astype(f)
    p = (cmax * (f(1) - s)).astype(f)
    q = (cmax * (f(1) - s * hf)).astype(f)
    t = (cmax * (f(1) - s * (f(1) - hf))).astype(f)
    v = cmax
    R = np.choose(hi % 6, [v, q, p, p, t, v])
    G = np.choose(hi % 6, [t, v, v, q, p, p])
    B = np.choose(hi % 6, [p, p, t, v, v, q])
    return np.stack([R, G, B], axis=1).astype(f) * f(alpha) + f(beta)


TWIST_SETS = [(1.0, 0.0, 0.0, 1.0), (0.9, 5.0, -18.0, 1.3), (1.4, -7.5, 18.0, 0.6), (0.6, 12.0, 123.0, 1.4), (1.17, 0.25, 301.5, 0.83)]


@pytest.mark.parametrize("alpha,beta,hue,sat", TWIST_SETS)
def test_color_twist_reciprocal_form_within_one_level_of_division_form_on_all_rgb(alpha, beta, hue, sat):
    # all 2^24 triples as one 4096 x 4096 image
    v = np.arange(1 << 24, dtype=np.uint32)
    rgb = np.stack([(v >> 16) & 255, (v >> 8) & 255, v & 255], axis=1).astype(np.uint8)
    img = rgb.reshape(1, 4096, 4096, 3)
    out = orc.color_twist(img, _full(1, 4096, 4096), [alpha], [beta], [hue], [sat]).reshape(-1, 3).astype(np.int32)
    worst, ndiff = 0, 0
    for lo in range(0, 1 << 24, 1 << 21):  # in slices: the float temporaries stay small
        ref = _twist_division_form(rgb[lo:lo + (1 << 21)], alpha, beta, hue, sat)
        exp = np.clip(np.rint(ref), 0, 255).astype(np.int32)
        d = np.abs(out[lo:lo + (1 << 21)] - exp)
        # a hue that lands exactly on a sector boundary in one form and a hair below it in the other changes the sector
        # but not the colour (both sectors give the same value there), so the level difference stays <= 1 as well
        worst = max(worst, int(d.max()))
        ndiff += int((d != 0).sum())
    print("colour twist (%g, %g, %g, %g): %d of %d values differ by one level" % (alpha, beta, hue, sat, ndiff, 3 << 24))
    assert worst <= 1
    assert ndiff < (3 << 24) * 0.02
    if (alpha, beta, hue, sat) == TWIST_SETS[0]:
        # identity parameters: the round trip reproduces every input triple to within one level
        assert np.abs(out - rgb.astype(np.int32)).max() <= 1


# ------------------------------------------------------------------ normalize: numpy statistics, hand-computed cases

def test_normalize_matches_numpy_statistics():
    rng = np.random.default_rng(31)
    n, h, w = 3, 20, 27
    img = _img(n, h, w, rng)
    roi = np.array([[0, 0, w, h], [3, 2, 11, 9], [5, 5, 1, 7]], np.uint32)
    for mask in (3, 7):
        out = orc.normalize(img, roi, axis_mask=mask, scale=2.0, shift=-0.5)
        for i in range(n):
            x0, y0, ww, hh = [int(v) for v in roi[i]]
            win = img[i, y0:y0 + hh, x0:x0 + ww].astype(np.float64)
            axes = (0, 1) if mask == 3 else (0, 1, 2)
            mu, sd = win.mean(axis=axes, keepdims=True), win.std(axis=axes, keepdims=True)  # population standard deviation
            with np.errstate(divide="ignore", invalid="ignore"):
                exp = np.where(sd > 0, (win - mu) / sd * 2.0 - 0.5, -0.5)
            assert np.abs(out[i, :hh, :ww] - exp).max() < 2e-4, (mask, i)
    # given statistics: one value, and one per channel
    out = orc.normalize(img, roi, mean=[100.0], stddev=[50.0])
    assert np.abs(out[0] - (img[0].astype(np.float64) - 100.0) / 50.0).max() < 1e-5
    out = orc.normalize(img, roi, mean=[10.0, 20.0, 30.0], stddev=[2.0, 4.0, 8.0], scale=3.0, shift=1.0)
    exp = (img[0].astype(np.float64) - [10.0, 20.0, 30.0]) / [2.0, 4.0, 8.0] * 3.0 + 1.0
    assert np.abs(out[0] - exp).max() < 1e-4
    # a given mean with a computed deviation: the deviation is taken around the GIVEN mean
    out = orc.normalize(img, roi[:1], mean=[0.0], axis_mask=7)
    rms = np.sqrt((img[0].astype(np.float64) ** 2).mean())
    assert np.abs(out[0] - img[0] / rms).max() < 1e-5


def test_normalize_hand_computed_cases():
    # constant image: deviation 0 -> every value becomes the shift
    img = np.full((1, 4, 6, 3), 77, np.uint8)
    out = orc.normalize(img, _full(1, 4, 6), shift=0.25)
    assert (out == 0.25).all()
    # half 10, half 30 in every channel: mean 20, deviation 10 -> -1 and +1 exactly
    img = np.empty((1, 4, 6, 3), np.uint8)
    img[:, :, :3] = 10
    img[:, :, 3:] = 30
    out = orc.normalize(img, _full(1, 4, 6))
    assert (out[0, :, :3] == -1.0).all() and (out[0, :, 3:] == 1.0).all()
    # channels 0 / 100 / 200, all axes: mean 100, deviation sqrt(20000/3)
    img = np.zeros((1, 2, 2, 3), np.uint8)
    img[..., 1], img[..., 2] = 100, 200
    out = orc.normalize(img, _full(1, 2, 2), axis_mask=7)
    assert np.allclose(out[0, 0, 0], [-100 / math.sqrt(20000 / 3), 0.0, 100 / math.sqrt(20000 / 3)], atol=1e-6)
    assert abs(out[0, 0, 0, 1]) < 1e-6  # fma(x, a, fma(-mean, a, 0)): the rounding of mean * a is all that is left
