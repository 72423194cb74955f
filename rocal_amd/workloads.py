"""Seeded synthetic workloads: the five benchmark configurations and the parameter laws that
feed them. Shared by the parity tests and the benchmark (no reference code is read at run time)."""
import math

import numpy as np

MEAN = np.array([123.675, 116.28, 103.53], np.float32)
STD = np.array([58.395, 57.12, 57.375], np.float32)


def smooth_noise(rng, n, h, w, sigma=3.0):
    """Gaussian-blurred uniform noise, requantised to u8 (contrast stretched back to 0..255)."""
    from scipy.ndimage import gaussian_filter
    out = np.empty((n, h, w, 3), np.uint8)
    for i in range(n):
        f = rng.random((h, w, 3), dtype=np.float32)
        f = gaussian_filter(f, sigma=(sigma, sigma, 0), mode="reflect")
        f = (f - f.min()) / max(float(f.max() - f.min()), 1e-6)
        out[i] = np.clip(np.rint(f * 255.0), 0, 255).astype(np.uint8)
    return out


def random_crop_dec_windows(master_seed, H, W, area=(0.08, 1.0), ratio=(3.0 / 4.0, 4.0 / 3.0), attempts=10):
    """Random-resized-crop windows (x, y, w, h per sample) drawn by the host layer's RocalRandomCropDecParam, the law of
    rocAL's fused decoders (rocAL/source/parameters/parameter_random_crop_decoder.cpp:42-112): per-sample engines seeded from
    seed_seq{master_seed}, area fraction uniform, aspect ratio log-uniform, rounded sides, ten attempts, fallback, uniform
    integer position."""
    import ctypes as C
    from . import backend
    n = len(H)
    hw = np.ascontiguousarray(np.stack([np.asarray(H), np.asarray(W)], axis=1), dtype=np.uint32)
    out = np.empty((n, 4), np.uint32)
    fn = backend.host().rocalpy_random_crop_dec_windows
    fn.restype = C.c_int
    fn.argtypes = [C.c_uint, C.c_uint, C.c_void_p, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, C.c_void_p]
    if fn(int(master_seed) & 0xFFFFFFFF, n, hw.ctypes.data, ratio[0], ratio[1], area[0], area[1], attempts, out.ctypes.data) != 0:
        raise RuntimeError("rocalpy_random_crop_dec_windows failed")
    return out


def config0(n=128, seed=1234):
    """CropMirrorNormalize: 256x256 u8 -> centre 224x224, fp32 NCHW."""
    rng = np.random.default_rng(seed)
    img = rng.integers(0, 256, (n, 256, 256, 3), dtype=np.uint8)
    crop = np.tile(np.array([16, 16, 224, 224], np.uint32), (n, 1))
    mirror = (rng.random(n) < 0.5).astype(np.uint32)
    return dict(img=img, crop=crop, mirror=mirror, out_h=224, out_w=224)


def config1(n=256, seed=1235, hw_range=(240, 640), sigma=3.0):
    """RandomResizedCrop + CMN, ragged batch -> 224x224 fp16 NCHW. Pixels: Gaussian-blurred uniform noise; windows: the
    decoder-side random-crop law with master seed `seed`."""
    rng = np.random.default_rng(seed)
    hmax = wmax = hw_range[1]
    H = rng.integers(hw_range[0], hw_range[1] + 1, n)
    W = rng.integers(hw_range[0], hw_range[1] + 1, n)
    img = np.zeros((n, hmax, wmax, 3), np.uint8)
    for i in range(n):
        img[i, :H[i], :W[i]] = smooth_noise(rng, 1, int(H[i]), int(W[i]), sigma)[0]
    roi = random_crop_dec_windows(seed, H, W)
    mirror = (rng.random(n) < 0.5).astype(np.uint32)
    return dict(img=img, roi=roi, mirror=mirror, out_h=224, out_w=224, H=H, W=W)


def config2(n=256, seed=1236):
    """ColorTwist on 224x224 u8."""
    rng = np.random.default_rng(seed)
    img = rng.integers(0, 256, (n, 224, 224, 3), dtype=np.uint8)
    roi = np.tile(np.array([0, 0, 224, 224], np.uint32), (n, 1))
    return dict(img=img, roi=roi,
                alpha=rng.uniform(0.6, 1.4, n).astype(np.float32),
                beta=rng.uniform(0.6, 1.4, n).astype(np.float32),
                hue=rng.uniform(-18.0, 18.0, n).astype(np.float32),
                sat=rng.uniform(0.6, 1.4, n).astype(np.float32))


def inverse_affine(theta_deg, scale, tx, ty):
    """dst->src matrix (about the centres) of: rotate by theta, scale by s, then translate by (tx,ty)."""
    t = math.radians(theta_deg)
    c, s = math.cos(t) / scale, math.sin(t) / scale
    # forward: d = s*R*p + t  =>  p = (1/s) R^T (d - t)
    m = np.array([[c, s, -(c * tx + s * ty)], [-s, c, -(-s * tx + c * ty)]], np.float32)
    return m


def config3(n=128, seed=1237, size=512, sigma=3.0):
    """WarpAffine: rotation +-30 deg, scale 0.9..1.1, translation +-16 px; u8 NHWC size x size."""
    rng = np.random.default_rng(seed)
    img = smooth_noise(rng, n, size, size, sigma)
    roi = np.tile(np.array([0, 0, size, size], np.uint32), (n, 1))
    affine = np.empty((n, 6), np.float32)
    for i in range(n):
        m = inverse_affine(rng.uniform(-30, 30), rng.uniform(0.9, 1.1), rng.uniform(-16, 16), rng.uniform(-16, 16))
        # rocAL's fill order: x0,y0,x1,y1,o0,o1 with M = [[x0,x1,o0],[y0,y1,o1]]
        affine[i] = [m[0, 0], m[1, 0], m[0, 1], m[1, 1], m[0, 2], m[1, 2]]
    return dict(img=img, roi=roi, affine=affine, out_h=size, out_w=size)


def config4(n=32, seed=1238, src_hw=(1080, 1920), dst_hw=(360, 640), sigma=3.0):
    """Triangular downscale of large images + normalise + mirror -> fp16 NCHW."""
    rng = np.random.default_rng(seed)
    h, w = src_hw
    img = smooth_noise(rng, n, h, w, sigma)
    sp = rng.random((n, h, w))
    img[sp < 0.025] = 0
    img[sp > 0.975] = 255
    roi = np.tile(np.array([0, 0, w, h], np.uint32), (n, 1))
    mirror = (rng.random(n) < 0.5).astype(np.uint32)
    return dict(img=img, roi=roi, mirror=mirror, out_h=dst_hw[0], out_w=dst_hw[1])
