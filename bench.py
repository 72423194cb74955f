#!/usr/bin/env python3
"""Benchmark of the augmentation hot path on one MI355X.

A step is one pass of the hot path over one batch: the launch that replaces vxProcessGraph for
the fused node (what rocAL's own process timer brackets). Inputs and the per-batch parameter
table are resident in HBM when the timed region starts. Prints ONE JSON line on stdout.

Every step reads a source batch and writes a destination batch that no earlier step of the last
gigabyte has touched: the timed loop rotates over K copies of the batch with K x (bytes per step)
>= 1 GiB, four times the 256 MB last-level cache, as a pipeline that gets a fresh batch per step
would. `value`, `ms_per_step` and `roofline.frac` are from that loop; `roofline.frac_warm` is the
same kernel replayed on ONE source/destination pair (which fits the cache) and is reported for
comparison only. Before anything is timed an untimed ramp of launches brings the GPU to its steady
clocks (config.clock_ramp_ms). config.update_ms_per_batch is the host time of the per-batch update
(parameter packing, launch planning, table upload) on fresh parameters, config.step_with_update_ms
one update + launch + wait per batch, as rocAL's output thread runs them
(rocAL/source/pipeline/master_graph.cpp:1010-1017).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 0..11] [--all] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published

WORKLOADS = {
    0: "C0 CropMirrorNormalize 256x256->224x224 fp32 NCHW batch 128 (configs[0])",
    1: "C1 RandomResizedCrop+CropMirrorNormalize ragged[240..640]->224x224 fp16 NCHW batch 256 (configs[1])",
    2: "C2 ColorTwist 224x224 u8->u8 NHWC batch 256 (configs[2])",
    3: "C3 WarpAffine 512x512 u8->u8 NHWC batch 128 (configs[3])",
    4: "C4 triangular 1920x1080->640x360 +normalize fp16 NCHW batch 32 (configs[4])",
    # the rows next to the path (measured with --all or --config; not the benchmark's configurations)
    5: "N1 ToTensor 224x224 u8 NHWC -> fp16 NCHW, reversed channels, batch 256",
    6: "N2 C1 (RandomResizedCrop+CropMirrorNormalize ->224x224 fp16 NCHW batch 256) reading a ragged, packed source (rows at dword pitch)",
    7: "N4 Gamma 224x224 u8->u8 NHWC batch 256",
    8: "N4 Blend of two batches 224x224 u8->u8 NHWC batch 256",
    9: "N4 Exposure 224x224 u8->u8 NHWC batch 256",
    10: "N4 ColorTemperature 224x224 u8->u8 NHWC batch 256",
    11: "C1 with a ColorTwist node fused between RandomResizedCrop and CropMirrorNormalize (one launch), ->224x224 fp16 NCHW batch 256",
    12: "C1's RandomResizedCrop windows with triangular (antialiasing) interpolation + normalize + mirror ->224x224 fp16 NCHW batch 256",
}


def build_case(cfg, ctx, n=None):
    """Returns (op, src_tensor, dst_tensor, n_images, cpu_fn, update_fn) for a configuration; cpu_fn(k) runs the
    CPU checker on the first k images of the same batch; update_fn(j) runs the op's per-batch update with the
    j-th fresh parameter set (j = 0: the set the timed launches use), or is None."""
    import torch
    from rocal_amd import ops, workloads as wl

    def scale_bias(k):
        inv = (1 / wl.STD).astype(np.float32)
        return np.tile(inv, k), np.tile(-(wl.MEAN * inv), k)

    if cfg == 0:
        n = n or 128
        c = wl.config0(n)
        scale, bias = scale_bias(n)
        op = ops.CropMirrorNormalize(ctx, ops.desc(n, 256, 256, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP32))
        def update(j):
            op.update(c["crop"], scale, bias, np.roll(c["mirror"], j))
        update(0)

        def cpu(k):
            from oracle import orc
            return orc.crop_mirror_normalize(c["img"][:k], c["crop"][:k], scale[:3 * k], bias[:3 * k], c["mirror"][:k], 224, 224, orc.NCHW, orc.FP32)
    elif cfg == 1:
        n = n or 256
        c = wl.config1(n)
        scale, bias = scale_bias(n)
        dw = np.full(n, 224, np.uint32)
        op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
        def update(j):  # j > 0: a fresh set of RandomResizedCrop windows and mirror flags for the same images
            if j == 0:
                op.update_cmn(c["roi"], dw, dw, scale, bias, c["mirror"])
            else:
                rng = np.random.default_rng(99000 + j)
                roi = wl.random_crop_dec_windows(99000 + j, c["H"], c["W"])
                op.update_cmn(roi, dw, dw, scale, bias, (rng.random(n) < 0.5).astype(np.uint32))
        update(0)

        def cpu(k):
            from oracle import orc
            return orc.resize(c["img"][:k], c["roi"][:k], dw[:k], dw[:k], 224, 224, interp=orc.LINEAR, mirror=c["mirror"][:k],
                              scale=scale[:3 * k], bias=bias[:3 * k], layout=orc.NCHW, dtype=orc.FP16, flags=orc.F_QUANTIZE_U8)
    elif cfg == 2:
        n = n or 256
        c = wl.config2(n)
        sd = ops.desc(n, 224, 224, ops.NHWC, ops.UINT8)
        op = ops.ColorTwist(ctx, sd, sd)
        def update(j):
            op.update(c["roi"], np.roll(c["alpha"], j), np.roll(c["beta"], j), np.roll(c["hue"], j), np.roll(c["sat"], j))
        update(0)

        def cpu(k):
            from oracle import orc
            return orc.color_twist(c["img"][:k], c["roi"][:k], c["alpha"][:k], c["beta"][:k], c["hue"][:k], c["sat"][:k])
    elif cfg == 3:
        n = n or 128
        c = wl.config3(n)
        sd = ops.desc(n, 512, 512, ops.NHWC, ops.UINT8)
        dw = np.full(n, 512, np.uint32)
        op = ops.WarpAffine(ctx, sd, sd, ops.LINEAR)
        def update(j):
            op.update(c["roi"], np.roll(c["affine"], j, axis=0), dw, dw)
        update(0)

        def cpu(k):
            from oracle import orc
            m = np.stack([orc.affine_from_rocal(a) for a in c["affine"][:k]])
            return orc.warp_affine(c["img"][:k], c["roi"][:k], m, dw[:k], dw[:k], 512, 512)
    elif cfg == 4:
        n = n or 32
        c = wl.config4(n)
        dw = np.full(n, 640, np.uint32)
        dh = np.full(n, 360, np.uint32)
        op = ops.Resize(ctx, ops.desc(n, 1080, 1920, ops.NHWC, ops.UINT8), ops.desc(n, 360, 640, ops.NCHW, ops.FP16), ops.TRIANGULAR)
        def update(j):
            op.update(c["roi"], dw, dh, np.roll(c["mirror"], j), np.tile(wl.MEAN, n), np.tile(wl.STD, n))
        update(0)
        scale, bias = scale_bias(n)

        def cpu(k):
            from oracle import orc
            return orc.resize(c["img"][:k], c["roi"][:k], dw[:k], dh[:k], 360, 640, interp=orc.TRIANGULAR, mirror=c["mirror"][:k],
                              scale=scale[:3 * k], bias=bias[:3 * k], layout=orc.NCHW, dtype=orc.FP16)
    elif cfg == 12:
        n = n or 256
        c = wl.config1(n)
        dw = np.full(n, 224, np.uint32)
        op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16), ops.TRIANGULAR)
        op.update(c["roi"], dw, dw, c["mirror"], np.tile(wl.MEAN, n), np.tile(wl.STD, n))
        scale, bias = scale_bias(n)

        def cpu(k):
            from oracle import orc
            return orc.resize(c["img"][:k], c["roi"][:k], dw[:k], dw[:k], 224, 224, interp=orc.TRIANGULAR, mirror=c["mirror"][:k],
                              scale=scale[:3 * k], bias=bias[:3 * k], layout=orc.NCHW, dtype=orc.FP16)
    elif cfg == 5:
        n = n or 256
        c = wl.config2(n)
        mul = (1 / wl.STD).astype(np.float32)
        add = (-(wl.MEAN / wl.STD)).astype(np.float32)
        op = ops.ToTensor(ctx, ops.desc(n, 224, 224, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16))
        op.update(mul, add, reverse_channels=True)

        def cpu(k):
            from oracle import orc
            return orc.to_tensor(c["img"][:k], mul, add, reverse_channels=True, layout=orc.NCHW, dtype=orc.FP16)
    elif cfg == 6:
        n = n or 256
        c = wl.config1(n)
        scale, bias = scale_bias(n)
        dw = np.full(n, 224, np.uint32)
        # the same images, one after the other, as a loader that writes dword-aligned rows packs them: every image starts at a
        # multiple of 4 bytes and its rows are padded to a multiple of 4 bytes (at most 3 bytes per row, 0.1 % of the batch)
        offsets, strides, parts, pos = [], [], [], 0
        for i in range(n):
            h, w = int(c["H"][i]), int(c["W"][i])
            st = (3 * w + 3) // 4 * 4
            rows = np.zeros((h, st), np.uint8)
            rows[:, :3 * w] = c["img"][i, :h, :w].reshape(h, 3 * w)
            offsets.append(pos)
            strides.append(st)
            parts.append(rows.reshape(-1))
            pos += h * st
        packed = np.concatenate(parts)
        op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16), ops.LINEAR, flags=ops.F_QUANTIZE_U8)
        op.set_ragged_source(np.array(offsets, np.uint64), c["W"], c["H"], packed.size, row_strides=strides)
        op.update_cmn(c["roi"], dw, dw, scale, bias, c["mirror"])

        padded, roi6, mirror6 = c["img"], c["roi"], c["mirror"]

        def cpu(k):
            from oracle import orc
            return orc.resize(padded[:k], roi6[:k], dw[:k], dw[:k], 224, 224, interp=orc.LINEAR, mirror=mirror6[:k],
                              scale=scale[:3 * k], bias=bias[:3 * k], layout=orc.NCHW, dtype=orc.FP16, flags=orc.F_QUANTIZE_U8)
        c = dict(img=packed)
    elif cfg == 11:
        n = n or 256
        c = wl.config1(n)
        tw = wl.config2(n)
        scale, bias = scale_bias(n)
        dw = np.full(n, 224, np.uint32)
        colour = (tw["alpha"], tw["beta"], tw["hue"], tw["sat"])
        op = ops.Resize(ctx, ops.desc(n, 640, 640, ops.NHWC, ops.UINT8), ops.desc(n, 224, 224, ops.NCHW, ops.FP16), ops.LINEAR,
                        flags=ops.F_QUANTIZE_U8 | ops.F_COLOR_TWIST)
        op.update_color_cmn(c["roi"], dw, dw, scale, bias, colour, c["mirror"])

        def cpu(k):  # the three reference nodes one after the other
            from oracle import orc
            mid = orc.resize(c["img"][:k], c["roi"][:k], dw[:k], dw[:k], 224, 224, interp=orc.LINEAR)
            whole = np.tile(np.array([0, 0, 224, 224], np.uint32), (k, 1))
            mid = orc.color_twist(mid, whole, *[p[:k] for p in colour])
            return orc.crop_mirror_normalize(mid, whole, scale[:3 * k], bias[:3 * k], c["mirror"][:k], 224, 224, orc.NCHW, orc.FP16)
    elif cfg in (7, 8, 9, 10):
        n = n or 256
        c = wl.config2(n)
        sd = ops.desc(n, 224, 224, ops.NHWC, ops.UINT8)
        rng = np.random.default_rng(4321 + cfg)
        img, roi = c["img"], c["roi"]
        if cfg == 7:
            p = rng.uniform(0.3, 7.0, n).astype(np.float32)  # the node's default range
            op = ops.Gamma(ctx, sd, sd)
            op.update(roi, p)
        elif cfg == 8:
            p = rng.uniform(0.1, 0.9, n).astype(np.float32)
            img2 = np.ascontiguousarray(img[::-1])
            op = ops.Blend(ctx, sd, sd)
            op.update(roi, p)
        elif cfg == 9:
            p = rng.uniform(0.15, 0.95, n).astype(np.float32)
            op = ops.Exposure(ctx, sd, sd)
            op.update(roi, p)
        else:
            p = rng.integers(-99, 100, n).astype(np.int32)
            op = ops.ColorTemperature(ctx, sd, sd)
            op.update(roi, p)

        def cpu(k):
            from oracle import orc
            if cfg == 7:
                return orc.gamma(img[:k], roi[:k], p[:k])
            if cfg == 8:
                return orc.blend(img[:k], img2[:k], roi[:k], p[:k])
            if cfg == 9:
                return orc.exposure(img[:k], roi[:k], p[:k])
            return orc.color_temperature(img[:k], roi[:k], p[:k])
        if cfg == 8:
            dst = op.alloc_output()
            return op, (torch.from_numpy(img).cuda(), torch.from_numpy(img2).cuda()), dst, n, cpu, None
    else:
        raise SystemExit("unknown config %r" % cfg)
    src = torch.from_numpy(c["img"]).cuda()
    dst = op.alloc_output()
    return op, src, dst, n, cpu, (update if cfg in (0, 1, 2, 3, 4) else None)


ROTATE_BYTES = 1 << 30   # the timed loop touches at least this much memory before it comes back to a buffer
RAMP_MS = 120.0          # untimed launches before anything is timed: the GPU reaches its steady clocks in ~35 ms


def _launcher(op, srcs, dst):
    if len(srcs) == 1:
        return op.prepared_launch(srcs[0], dst)
    return lambda: op.launch(*srcs, dst)


def clock_ramp(launchers, min_ms=RAMP_MS):
    """Untimed launches (cycling through the buffer pairs) for at least min_ms of wall time; returns (launches, ms)."""
    import torch
    t0 = time.perf_counter()
    count = 0
    while (time.perf_counter() - t0) * 1e3 < min_ms:
        for _ in range(200):
            launchers[count % len(launchers)]()
            count += 1
        torch.cuda.synchronize()
    return count, (time.perf_counter() - t0) * 1e3


def time_loop(launchers, steps, warmup):
    """`steps` launches, cycling through `launchers`, between two HIP events recorded on the stream the kernels run
    on (the context borrows torch's current stream). Returns (ms per launch on the device, ms per step by the host clock)."""
    import torch
    k = len(launchers)
    for i in range(warmup):
        launchers[i % k]()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        launchers[i % k]()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return e0.elapsed_time(e1) / steps, wall * 1e3 / steps


def time_updates(op, update_fn, launchers, steps, sets=12):
    """Host cost of the per-batch update on fresh parameters, and of whole steps that include it."""
    import torch
    calls = []
    for j in range(1, sets + 1):
        update_fn(j)
        calls.append(op.prepared_update())
    update_fn(0)
    calls.append(op.prepared_update())  # the last one restores the parameters of the timed launches
    torch.cuda.synchronize()
    # (a) the update alone: packs, plans, starts the table upload; nothing waits for the GPU
    t = []
    for rep in range(5):
        for c in calls:
            t0 = time.perf_counter()
            c()
            t.append(time.perf_counter() - t0)
        torch.cuda.synchronize()
    update_ms = float(np.median(t)) * 1e3
    # (b) update -> launch -> wait, one batch at a time, as rocAL's output thread runs them
    k, m = len(launchers), len(calls)
    nsteps = max(steps, 200)
    for i in range(20):
        calls[i % m]()
        launchers[i % k]()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(nsteps):
        calls[i % m]()
        launchers[i % k]()
        torch.cuda.synchronize()
    serial_ms = (time.perf_counter() - t0) * 1e3 / nsteps
    # (c) the same without waiting per batch: the 4-slot table ring lets the host run ahead of the GPU
    t0 = time.perf_counter()
    for i in range(nsteps):
        calls[i % m]()
        launchers[i % k]()
    torch.cuda.synchronize()
    piped_ms = (time.perf_counter() - t0) * 1e3 / nsteps
    calls[-1]()
    torch.cuda.synchronize()
    return update_ms, serial_ms, piped_ms


def stream_ceilings(ctx, nbytes=1 << 30, reps=12):
    """What the memory system of this box gives a kernel with no arithmetic, on 1 GiB buffers (four times the last-level
    cache): a copy (bytes read + bytes written per second), a pass that only reads and one that only writes, each the best
    over 4 / 8 / 16 / 32 workgroups per compute unit of the library's streaming probe. GB/s."""
    import torch
    a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    b = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    a.zero_()
    b.zero_()
    out = {}
    for mode, name, factor in ((0, "copy", 2.0), (1, "read_only", 1.0), (2, "write_only", 1.0)):
        best = (0.0, 0)
        for g in (4, 8, 16, 32):
            for _ in range(3):
                ctx.stream_probe(mode, a, b, nbytes, g)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                ctx.stream_probe(mode, a, b, nbytes, g)
            e1.record()
            torch.cuda.synchronize()
            rate = factor * nbytes / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9
            best = max(best, (rate, g))
        out[name] = best
    del a, b
    torch.cuda.empty_cache()
    return out


def rocal_protocol(batches=400, pairs=4):
    """C1 through the reference's own entry points, as a rocAL program runs a batch: rocalCreate -> rocalDeviceSource ->
    rocalCropResize (random windows, renewed per batch by the C++ ParameterFactory) -> rocalCropMirrorNormalize (random mirror)
    -> rocalVerify; the two nodes run as one launch. Sources and destinations rotate over `pairs` buffers (4 x 315 MB of
    padded sources). Returns milliseconds per batch:
      serial     feed, rocalRun, rocalGetOutputTensors (the consumer's wait) for every batch, by the host clock;
      pipelined  the same without the per-batch wait (one wait at the end): the host runs ahead of the GPU;
      process / update  the library's own timers for the serial loop (rocalGetTimingInfo().process_time: launches + the wait;
                 rocalGetParameterUpdateTime: parameter renewal + node updates), per batch."""
    import torch
    from rocal_amd import fn, types, workloads as wl
    from rocal_amd.pipeline import Pipeline, b
    n = 256
    c = wl.config1(n)
    pipe = Pipeline(batch_size=n, device_id=0, seed=1235)
    with pipe:
        src = pipe.device_source(640, 640)
        a = fn.resize_crop(src, resize_width=224, resize_height=224)
        out = fn.crop_mirror_normalize(a, crop=(224, 224), mean=[float(x) for x in wl.MEAN], std=[float(x) for x in wl.STD],
                                       mirror=b.createIntRand([0, 1], [0.5, 0.5], 2), output_layout=types.NCHW, output_dtype=types.FLOAT16)
        pipe.set_outputs(out)
    pipe.build()
    srcs = [torch.from_numpy(c["img"]).cuda() for _ in range(pairs)]
    dsts = [torch.empty((n, 3, 224, 224), dtype=torch.float16, device="cuda") for _ in range(pairs)]
    import numpy as np
    W, H = np.ascontiguousarray(c["W"], dtype=np.uint32), np.ascontiguousarray(c["H"], dtype=np.uint32)

    def one(i, wait):
        pipe.feed(src, srcs[i % pairs], W, H)
        pipe.bind_output(out, dsts[i % pairs])
        pipe.rocal_run()
        if wait:
            pipe.get_output_tensors()
    for i in range(50):
        one(i, True)
    pipe.timing_info()
    t0 = time.perf_counter()
    for i in range(batches):
        one(i, True)
    serial = (time.perf_counter() - t0) * 1e3 / batches
    t = pipe.timing_info()
    t0 = time.perf_counter()
    for i in range(batches):
        one(i, False)
    pipe.get_output_tensors()
    piped = (time.perf_counter() - t0) * 1e3 / batches
    pipe.release()
    del srcs, dsts
    torch.cuda.empty_cache()
    return {"serial": serial, "pipelined": piped, "process": t["process_time"] * 1e-3 / batches, "update": t["parameter_update_time"] * 1e-3 / batches}


def cpu_baseline(cpu_fn, n, budget_s=12.0):
    """Times the CPU checker (a port of the reference semantics, OpenMP over samples) on a bounded
    sample of the same batch."""
    from oracle import orc
    k = min(n, 16)
    cpu_fn(k)  # first call pays for the thread pool and page faults
    t0 = time.perf_counter()
    cpu_fn(k)
    dt = time.perf_counter() - t0
    per_img = dt / k
    k2 = int(max(k, min(n, budget_s / max(per_img, 1e-9))))
    reps = max(1, int(round(budget_s / max(per_img * k2, 1e-9))))
    t0 = time.perf_counter()
    for _ in range(reps):
        cpu_fn(k2)
    dt = time.perf_counter() - t0
    return {"value": round(k2 * reps / dt, 1), "unit": "images/s", "cores": orc.num_threads(), "kind": "port",
            "sample": "%d images of the same batch x %d passes (%.1f s)" % (k2, reps, dt)}


def measured_traffic(cfg, kernel):
    """HBM bytes per launch of this configuration's kernel, from the committed rocprofv3 counter
    summaries (FETCH_SIZE + WRITE_SIZE, each scaled by the same counter's reading for a plain
    1 GiB copy). None when no summary covers the kernel that runs now."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            rec = json.load(f).get(str(cfg))
    except OSError:
        return None
    if not rec or rec.get("kernel") != kernel:
        return None
    return rec["fetch_bytes"] + rec["write_bytes"]


def run_config(cfg, ctx, steps, warmup, with_cpu, rotating_only=False, ramp_ms=RAMP_MS, resident_only=False):
    import torch
    op, src, dst, n, cpu_fn, update_fn = build_case(cfg, ctx)
    srcs = src if isinstance(src, tuple) else (src,)
    algo = op.algorithmic_bytes
    # K source/destination pairs at different addresses: K x (bytes a step touches) >= 1 GiB
    copies = max(2, -(-ROTATE_BYTES // max(algo, 1)))
    pairs = [(srcs, dst)] + [(tuple(t.clone() for t in srcs), torch.empty_like(dst)) for _ in range(copies - 1)]
    launchers = [_launcher(op, sp, d) for sp, d in pairs]
    if resident_only:  # (counter and trace runs of the cache-resident regime: every launch of the process replays one pair)
        launchers = launchers[:1]
    ramp_launches, ramp_ms = clock_ramp(launchers, ramp_ms) if ramp_ms > 0 else (0, 0.0)
    ms_kernel, ms_step = time_loop(launchers, steps, warmup)          # rotating: the reported figure
    ms_warm = ms_kernel
    if not rotating_only and not resident_only:
        ms_warm, _ = time_loop(launchers[:1], steps, warmup)          # one pair, cache-resident: for comparison
    achieved = algo / (ms_kernel * 1e-3) / 1e9
    warm = algo / (ms_warm * 1e-3) / 1e9
    out = {
        "metric": "images/s", "value": round(n / (ms_kernel * 1e-3), 1), "unit": "images/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": round(ms_kernel, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": WORKLOADS[cfg], "batch": n, "kernel": op.kernel_name, "algorithmic_bytes_per_launch": algo, "plan": op.plan,
                   "host_ms_per_step": round(ms_step, 6), "rotating_buffer_pairs": copies,
                   "clock_ramp_ms": round(ramp_ms, 1), "clock_ramp_launches": ramp_launches,
                   "ms_per_step_warm": round(ms_warm, 6)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(cfg, op.kernel_name),
                     "achieved_warm": round(warm, 1), "frac_warm": round(warm / HBM_PEAK_GBPS, 4)},
    }
    if rotating_only or resident_only:
        out["config"]["regime"] = "rotating" if rotating_only else "resident (one buffer pair replayed: NOT the benchmark's figure)"
        for k in ("ms_per_step_warm",):
            out["config"].pop(k)
        for k in ("achieved_warm", "frac_warm"):
            out["roofline"].pop(k)
    if update_fn is not None and not rotating_only and not resident_only:
        upd, serial, piped = time_updates(op, update_fn, launchers, steps)
        out["config"]["update_ms_per_batch"] = round(upd, 6)
        out["config"]["step_with_update_ms"] = round(serial, 6)
        out["config"]["step_with_update_pipelined_ms"] = round(piped, 6)
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline(cpu_fn, n)
    del op, src, dst, srcs, pairs, launchers
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # After an idle spell (building the synthetic batch takes seconds of host time) the GPU needs about a thousand
    # launches (~35 ms) to reach its steady clocks; an untimed ramp of launches (clock_ramp) covers that whatever
    # --warmup says. The default timed region is long enough for the profiler's average over all launches to agree.
    ap.add_argument("--steps", type=int, default=6000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--config", type=int, default=1)
    ap.add_argument("--all", action="store_true", help="also measure the other configurations (one JSON object per configuration on stderr, and all of them in the file --all-out names)")
    ap.add_argument("--all-out", default=None, help="with --all: file that receives every configuration's result as one JSON object")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--rotating-only", action="store_true", help="only the ramp and the rotating timed loop: every launch of the process is of the "
                    "reported kind, so a rocprofv3 kernel summary of this command averages the same thing")
    ap.add_argument("--resident-only", action="store_true", help="only the ramp and a timed loop that replays ONE buffer pair (the cache-resident "
                    "regime, for profiler and counter runs; not the benchmark's figure)")
    ap.add_argument("--ramp-ms", type=float, default=RAMP_MS, help="length of the untimed clock ramp (0 for counter runs, which only count)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py: this build measures ONE GPU (the path shards trivially by sample; no multi-GPU figure is produced). "
                         "Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    from rocal_amd import ops
    ctx = ops.Context(0)
    streams = stream_ceilings(ctx)
    ceiling = streams["copy"][0]
    res = run_config(args.config, ctx, args.steps, args.warmup, not args.no_cpu and not args.rotating_only and not args.resident_only,
                     args.rotating_only, args.ramp_ms, args.resident_only)
    res["metric"] = "images/s + HBM GB/s (% peak), RandomResizedCrop+CMN 224^2 fp16, batch 256" if args.config == 1 else "images/s"
    res["roofline"]["copy_ceiling_GBps"] = round(ceiling, 1)
    res["roofline"]["frac_of_copy_ceiling"] = round(res["roofline"]["achieved"] / ceiling, 4)
    res["roofline"]["read_only_GBps"] = round(streams["read_only"][0], 1)
    res["roofline"]["write_only_GBps"] = round(streams["write_only"][0], 1)
    res["roofline"]["stream_probe_groups_per_cu"] = {k: v[1] for k, v in streams.items()}
    if args.config == 1 and not args.rotating_only and not args.resident_only:
        rp = rocal_protocol()
        res["config"]["rocal_run_ms_per_batch"] = round(rp["process"] + rp["update"], 6)
        res["config"]["rocal_run_process_ms"] = round(rp["process"], 6)
        res["config"]["rocal_run_update_ms"] = round(rp["update"], 6)
        res["config"]["rocal_run_host_ms_per_batch"] = round(rp["serial"], 6)
        res["config"]["rocal_run_pipelined_ms_per_batch"] = round(rp["pipelined"], 6)
    if args.all:
        allres = {args.config: res}
        for cfg in sorted(WORKLOADS):
            if cfg != args.config:
                allres[cfg] = run_config(cfg, ctx, args.steps, args.warmup, not args.no_cpu and not args.rotating_only, args.rotating_only, args.ramp_ms)
                allres[cfg]["roofline"]["copy_ceiling_GBps"] = round(ceiling, 1)
                print("config %d: %s" % (cfg, json.dumps(allres[cfg])), file=sys.stderr)
        if args.all_out:
            os.makedirs(os.path.dirname(os.path.abspath(args.all_out)), exist_ok=True)
            with open(args.all_out, "w") as f:
                json.dump(allres, f, indent=1)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
