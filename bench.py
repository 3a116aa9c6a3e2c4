#!/usr/bin/env python3
"""Benchmark of the Deep8 dense-contraction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--no-cpu] [--no-others] [--settle-ms 60]

A step is one forward + both backward passes of the workload over one batch of synthetic input that
already sits in HBM.  The headline workload is benchmark configuration 3 (MatrixMultiply, half,
4096 x 4096 x 4096); the other configs are timed briefly and reported under "others".
Prints ONE JSON line.

Every measurement is preceded by --settle-ms (default 60) milliseconds of the same work, untimed: the chip's
power management raises the shader clock over the first 35-50 milliseconds of sustained load, so a run that
starts on an idle device and times 20 steps after 3 warm-up steps measures the ramp, not the rate a training
loop sees (MatrixMultiply half 4096^3: about 1185 TFLOP/s from idle, about 1425 sustained, same box, same
binary).  --settle-ms 0 gives the from-idle number; the JSON line reports the value used as "settle_ms".

  value          whole-step throughput: algorithmic FLOPs of fwd + dX + dY / wall time of a step.  A step is what this
                 build's executor issues: the forward product, then both gradient products in their overwrite form
                 (the executor's zero fill of a gradient is deferred until something reads it; --eager-zero times
                 the reference executor's literal fill + accumulate instead, and the line always carries it beside
                 the headline as "eager_zero")
  roofline       flops of one product / the average duration per product of the step's launches, each launch timed
                 alone with HIP events on the stream it runs on, against the dense MFMA peak of the element type
                 (element-wise and pooling workloads: the longest kernel's bytes / its duration, against HBM)
  cpu_baseline   Deep8's own CPU (Eigen) path from oracle/_ref -- or the C restatement when that was
                 not built -- on a bounded sample of the same workload, on this host's cores
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"f16": 2500.0, "f32": 157.3, "f64": 78.6}   # dense MFMA TFLOP/s, MI355X
HBM_PEAK = 8000.0                      # GB/s
# --eager-zero: fill both gradients and accumulate into them (the reference executor's literal sequence)
EAGER_ZERO = False

# HBM-side bytes per launch of the dominant kernel: read from the "HBM-side traffic per dispatch" table of the
# rocprofv3 summary kept under profiles/ for the workload (FETCH_SIZE / WRITE_SIZE runs of this file, each counter
# scaled by what it reads for a plain copy of known size).  workload -> (summary, rows of the table that make
# up one launch of the roofline kernel: substrings of the kernel column, each with the number of dispatches
# of that row per launch; a list of alternatives is averaged).  None where the summary or a row is missing.
TRAFFIC_ROWS = {
    "c3": ("gemm_wide_f16_matmul_4096_half.txt", [("gemm_wide_kernel", 1.0 / 3)]),           # NN, NT, TN averaged
    "f1": ("gemm_tiled_pair_f16_matmul_1024_half.txt", [("2x2 waves, NN>", 1.0 / 3), ("gemm_tiled_pair_kernel", 1.0 / 3)]),  # fwd + the gradients' shared launch, per product
    "c4": ("conv2d_fp32_b32_56x56x64_3x3.txt", [("NT, A = patch rows", 1), ("gemm_split_reduce", 1)]),  # forward: one launch (remainder band included) + the band's reduction
    "c5": ("deconv2d_half_b16_28x28x128_4x4s2.txt", [("one class of output pixels", 1)]),    # forward: one launch over the classes
    "d3": ("gemm_f64_matmul_2048_double.txt", [("gemm_f64_kernel", 1.0 / 3)]),
    "e4": ("elementwise_bias_relu_b32_56x56x64.txt", {"add (bias broadcast)": [("add_kernel", 1)], "relu": [("relu_kernel", 1)],
                                                       "relu_grad": [("relu_grad_kernel", 1)],
                                                       "bias_grad (sum over rows)": [("column_sum_kernel", 1), ("column_sum_finish", 1)]}),
    "p4": ("maxpool2d_b32_56x56x64.txt", {"maxpool2d": [("pool_forward_kernel", 1)], "maxpool2d_grad": [("pool_backward", 1)]}),
    "k5": ("deconv_maps_half_b16_28x28_to_56x56x64_4x4s2.txt", {"deconv_im2col": [("deconv_im2col_blocks_kernel", 1)],
                                                                 "deconv_col2im": [("deconv_col2im_lds_kernel", 1)]}),
    "i4": ("im2col_col2im_fp32_b32_56x56x64_3x3.txt", {"im2col": [("im2col_vec_kernel", 1)], "col2im": [("col2im_kernel", 1)]}),
}


def profile_traffic(key, part=None):
    """{"bytes": fetch + write bytes per launch, "source": file} from the committed summary, or None"""
    ent = TRAFFIC_ROWS.get(key)
    if ent is None:
        return None
    fname, rows = ent
    if isinstance(rows, dict):
        rows = rows.get(part)
        if rows is None:
            return None
    path = os.path.join(ROOT, "profiles", fname)
    if not os.path.exists(path):
        return None
    table, seen = [], False
    for line in open(path):
        if line.startswith("HBM-side traffic per dispatch"):
            seen = True
            continue
        if seen:
            f = line.split(None, 4)
            if len(f) == 5 and f[0].replace(".", "").isdigit():
                table.append((float(f[1]), float(f[3]), f[4].strip()))  # fetch MiB, write MiB, kernel
    total = 0.0
    for sub, count in rows:
        hit = [t for t in table if sub in t[2]]
        if not hit:
            return None
        total += count * sum(t[0] + t[1] for t in hit) * 2**20
    return {"bytes": int(total), "source": "profiles/" + fname}


def _traffic_fields(key, part=None):
    t = profile_traffic(key, part)
    return {"traffic": t["bytes"] if t else None, "traffic_source": t["source"] if t else None}


def _dev(a):
    from deep8_amd.capi import DeviceArray
    return DeviceArray.from_numpy(a)


# Milliseconds of untimed, uninterrupted work issued before every measurement (--settle-ms).  The chip's power
# management raises the shader clock over the first tens of milliseconds of sustained load: a measurement that
# starts on an idle device runs its first steps 15-20 % slower than the sustained rate (by the fp16 kernel's own
# clock record 1.4 GHz after 4 ms of load, 1.65 GHz after 40 ms), and a few warm-up steps do not cover that ramp.
SETTLE_MS = 60.0


def _settle(fn):
    """keeps the device busy with fn for SETTLE_MS of wall time, untimed.  The loop is bounded by the clock, not
    by a call count derived from one timed call: the first call of an entry point in a process also loads its
    code object, which would make that estimate far too small."""
    from deep8_amd import capi
    if SETTLE_MS <= 0:
        return
    fn()
    capi.sync()
    t0 = time.perf_counter()
    fn()
    capi.sync()
    one = max(time.perf_counter() - t0, 1e-6)
    burst = max(1, min(64, int(2e-3 / one)))  # about 2 ms of work between two looks at the clock
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(burst):
            fn()
        capi.sync()


REPS = 5   # --reps: the timed region (exactly --steps steps) is repeated this often; the median is reported


def _time_steps(fn, steps, warmup, reps=None):
    """wall-clock ms per step over exactly `steps` calls, device idle on both sides; the region is timed
    `reps` times back to back (the device stays under load in between) and the median is returned together
    with every sample"""
    from deep8_amd import capi
    _settle(fn)
    samples = []
    for _ in range(reps or REPS):
        for _ in range(warmup):
            fn()
        capi.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        capi.sync()
        samples.append((time.perf_counter() - t0) * 1e3 / steps)
    return float(np.median(samples)), samples


def _time_events(fn, reps):
    """average ms per call measured with HIP events on the launch stream"""
    from deep8_amd import capi
    _settle(fn)
    fn()
    capi.sync()
    t = capi.Timer(None)
    t.start()
    for _ in range(reps):
        fn()
    return t.stop_ms() / reps


class MatMulWorkload:
    """MatrixMultiply forward + GradX + GradY through d8_matmul* (Math::MatrixMultiply*GPU)."""

    def __init__(self, name, dtype, xs, ys, gen, seed):
        from deep8_amd import capi
        self.name, self.dtype = name, np.dtype(dtype)
        self.lib = capi.init()
        self.stream = None  # a hipStream_t as an integer, or None for the default stream
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        self.xs, self.ys = xs, ys
        zb = max(xs[0], ys[0])
        self.zs = (zb, xs[1], ys[2])
        self.x, self.y, self.dz = _dev(gen["x"](r, xs).astype(dtype)), _dev(gen["y"](r, ys).astype(dtype)), \
            _dev(gen["dz"](r, self.zs).astype(dtype))
        self.z = capi.DeviceArray(self.zs, dtype)
        self.dx = capi.DeviceArray(xs, dtype)
        self.dy = capi.DeviceArray(ys, dtype)
        nb = max(self.lib.d8_matmul_scratch_bytes(self.dt, w, *xs, *ys) for w in range(4))  # (3: both gradients from one call)
        self.ws_bytes = nb
        self.ws = capi.DeviceArray((max(nb, 16),), np.uint8)
        m, k, n = xs[1], xs[2], ys[2]
        self.flops = 3 * 2.0 * zb * m * k * n
        wide = self.dtype == np.float16 and m >= 256 and n >= 256 and k % 64 == 0 and zb * (-(-m // 256)) * (-(-n // 256)) >= 192
        small = zb * (-(-m // 128)) * (-(-n // 128)) <= 4 and max(m, n, k) * (zb if 1 in (xs[0], ys[0]) else 1) <= 512
        self.kernel = "%s (%s)" % (
            "gemm_f64_kernel (%s tiles, v_mfma_f64_16x16x4_f64)" % ("128x128" if zb * (-(-m // 128)) * (-(-n // 128)) >= 192 else "64x64")
            if self.dtype == np.float64 else
            "gemm_wide_kernel (fp16, 256x256 tiles)" if wide else
            "gemm_%s_kernel<%s>" % ("small" if small else "tiled", "f16" if self.dtype == np.float16 else "f32"),
            "one launch for fwd, one for dX and dY together" if wide or small or zb * (-(-m // 128)) * (-(-k // 128)) + (-(-k // 128)) * (-(-n // 128)) <= 128
            else "one launch each for fwd, dX, dY")
        es = self.dtype.itemsize
        nx, ny, nz = np.prod(xs), np.prod(ys), np.prod(self.zs)
        # fwd reads x,y writes z; dX reads dz,y and read-modify-writes dx; dY likewise
        self.bytes = es * ((nx + ny + nz) + (nz + ny + 2 * nx) + (nx + nz + 2 * ny))

    def fwd(self):
        from deep8_amd.capi import check
        check(self.lib.d8_matmul(self.dt, self.x.ptr, *self.xs, self.y.ptr, *self.ys, self.z.ptr,
                                 self.ws.ptr, self.ws_bytes, self.stream))

    def grad_x(self):
        from deep8_amd.capi import check
        check(self.lib.d8_matmul_grad_x(self.dt, self.dx.ptr, *self.xs, self.y.ptr, *self.ys, self.dz.ptr,
                                        self.ws.ptr, self.ws_bytes, self.stream))

    def grad_y(self):
        from deep8_amd.capi import check
        check(self.lib.d8_matmul_grad_y(self.dt, self.x.ptr, *self.xs, self.dy.ptr, *self.ys, self.dz.ptr,
                                        self.ws.ptr, self.ws_bytes, self.stream))

    def grad_x_first(self):
        from deep8_amd.capi import check
        check(self.lib.d8_matmul_grad_x_overwrite(self.dt, self.dx.ptr, *self.xs, self.y.ptr, *self.ys, self.dz.ptr,
                                                  self.ws.ptr, self.ws_bytes, self.stream))

    def grad_y_first(self):
        from deep8_amd.capi import check
        check(self.lib.d8_matmul_grad_y_overwrite(self.dt, self.x.ptr, *self.xs, self.dy.ptr, *self.ys, self.dz.ptr,
                                                  self.ws.ptr, self.ws_bytes, self.stream))

    def grad_xy(self, overwrite):
        """both gradients from one call, as MatrixMultiply::backward() of the host layer issues them"""
        from deep8_amd.capi import check
        check(self.lib.d8_matmul_grad_xy(self.dt, self.x.ptr, self.dx.ptr, *self.xs, self.y.ptr, self.dy.ptr, *self.ys,
                                         self.dz.ptr, 3 if overwrite else 0, self.ws.ptr, self.ws_bytes, self.stream))

    def grad_xy_first(self):
        self.grad_xy(True)

    def grad_xy_accumulate(self):
        self.grad_xy(False)

    def step(self):
        """One forward + backward of a MatrixMultiply node as this build's executor issues it: forward, then the
        two gradient products from one call.  The executor's zeroGradient() before a backward pass is deferred
        (Device::zeroLater), so the first product into each gradient is the overwrite form: same
        result as fill + accumulate, without the fill and without reading the zeros back."""
        if EAGER_ZERO:
            return self.step_eager_zero()
        self.fwd()
        self.grad_xy(True)

    def step_eager_zero(self):
        """The reference executor's literal sequence (deep8/src/model/EagerExecutor.cpp:51-65, then
        MatrixMultiply.cu:203 with beta = 1): forward, fill both gradients with zeros, accumulate into them."""
        self.fwd()
        self.dx.zero_()
        self.dy.zero_()
        self.grad_xy(False)

    def parts(self):
        """the calls of a step, each alone: the forward product, and both gradients from one call (for large Float16
        products one launch); beside them each gradient product as a call of its own"""
        f = self.flops / 3
        if EAGER_ZERO:
            return {"fwd": (self.fwd, f), "grad_xy": (self.grad_xy_accumulate, 2 * f), "grad_x": (self.grad_x, f), "grad_y": (self.grad_y, f)}
        return {"fwd": (self.fwd, f), "grad_xy": (self.grad_xy_first, 2 * f), "grad_x": (self.grad_x_first, f), "grad_y": (self.grad_y_first, f)}

    def parts_accumulate(self):
        """the gradient launches in their beta = 1 form (read the destination, add, write)"""
        f = self.flops / 3
        return {"grad_xy_accumulate": (self.grad_xy_accumulate, 2 * f), "grad_x_accumulate": (self.grad_x, f),
                "grad_y_accumulate": (self.grad_y, f)}


def mfma_stream_ceiling(wl, dtype_name):
    """TFLOP/s of back-to-back MFMAs on this workload's own operand bits (registers only, no LDS or
    global traffic): the matrix pipe's sustained rate under the power limit, which depends on the
    data.  Timed with HIP events like the GEMM launches."""
    import ctypes
    from deep8_amd import capi
    lib = wl.lib
    out = capi.DeviceArray((lib.d8_mfma_stream_out_bytes(),), np.uint8)
    flops = ctypes.c_double(0)
    iters = {2: 200, 4: 100, 8: 1000}[wl.dtype.itemsize]  # 100-400 us per launch, like the GEMMs

    def run():
        capi.check(lib.d8_mfma_stream(wl.dt, wl.x.ptr, wl.x.nbytes, out.ptr, iters, ctypes.byref(flops), None))
    for _ in range(10):
        run()
    ms = _time_events(run, 30)
    t = flops.value / (ms * 1e-3) / 1e12
    return {"tflops": round(t, 1), "frac_of_peak": round(t / PEAK[dtype_name], 4), "launch_us": round(ms * 1e3, 1),
            "operands": "x of this workload", "note": "MFMA instructions only, operands in registers"}


class ConvWorkload:
    """Conv2d or DeConv2d forward + GradX + GradY through d8_conv2d* / d8_deconv2d*."""

    def __init__(self, name, dtype, deconv, B, IH, IW, IC, OC, FH, FW, covered, sy, sx, seed, explicit=False):
        from deep8_amd import capi, ops
        self.name, self.dtype, self.deconv = name, np.dtype(dtype), deconv
        # explicit: the reference's own lowering (im2col -> GEMM, GEMM -> col2im through the interim matrix);
        # the library reads D8_CONV_EXPLICIT at every call
        self.explicit = explicit
        self.stream = None  # a hipStream_t as an integer, or None for the default stream
        if explicit:
            os.environ["D8_CONV_EXPLICIT"] = "1"
        self.key = name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        self.B = B
        r = np.random.default_rng(seed)
        if deconv:
            OH, OW, _, _ = ops.deconv2d_geometry(IH, IW, FH, FW, covered, sy, sx)
            self.geo = (int(covered), sy, sx)
        else:
            OH, OW, _, _ = ops.conv2d_geometry(IH, IW, FH, FW, covered, sy, sx, 1, 1)
            self.geo = (int(covered), sy, sx, 1, 1)
        self.xd, self.wd = (B, IH, IW, IC), (OC, FH, FW, IC)
        self.x = _dev(r.standard_normal((B, IH, IW, IC)).astype(np.float32).astype(dtype))
        self.w = _dev((r.standard_normal((OC, FH, FW, IC)) * np.sqrt(2.0 / (FH * FW * IC))).astype(np.float32).astype(dtype))
        self.gz = _dev(r.standard_normal((B, OH, OW, OC)).astype(np.float32).astype(dtype))
        self.z = capi.DeviceArray((B, OH, OW, OC), dtype)
        self.gx = capi.DeviceArray((B, IH, IW, IC), dtype)
        self.gw = capi.DeviceArray((OC, FH, FW, IC), dtype)
        q = self.lib.d8_deconv2d_scratch_bytes if deconv else self.lib.d8_conv2d_scratch_bytes
        self.ws_bytes = max(q(self.dt, w, B, IH, IW, IC, OC, FH, FW, *self.geo) for w in range(4))  # (3: both gradients from one call)
        self.ws = capi.DeviceArray((max(self.ws_bytes, 16),), np.uint8)
        os.environ.pop("D8_CONV_EXPLICIT", None)
        if deconv:
            self.flops = 3 * 2.0 * (B * IH * IW) * IC * (OC * FH * FW)
            mat = B * IH * IW * OC * FH * FW
        else:
            self.flops = 3 * 2.0 * (B * OH * OW) * (FH * FW * IC) * OC
            mat = B * OH * OW * FH * FW * IC
        es = self.dtype.itemsize
        nx, nw, nz = B * IH * IW * IC, OC * FH * FW * IC, B * OH * OW * OC
        self.mat_bytes = mat * es
        # operator-level algorithmic bytes: each pass reads its two operands and writes (forward) or
        # reads and writes (gradients) its result; the interim matrix is an implementation detail
        self.bytes = es * ((nx + nw + nz) + (nz + nw + 2 * nx) + (nx + nz + 2 * nw))

    def _call(self, fn, a, b, c):
        from deep8_amd.capi import check
        B, IH, IW, IC = self.xd
        OC, FH, FW, _ = self.wd
        if self.explicit:
            os.environ["D8_CONV_EXPLICIT"] = "1"
        try:
            check(fn(self.dt, a, B, IH, IW, IC, b, OC, FH, FW, c, *self.geo, self.ws.ptr, self.ws_bytes, self.stream))
        finally:
            if self.explicit:
                os.environ.pop("D8_CONV_EXPLICIT", None)

    def fwd(self):
        self._call(self.lib.d8_deconv2d if self.deconv else self.lib.d8_conv2d, self.x.ptr, self.w.ptr, self.z.ptr)

    def grad_x(self):
        first = "" if EAGER_ZERO else "_overwrite"
        self._call(getattr(self.lib, ("d8_deconv2d_grad_x" if self.deconv else "d8_conv2d_grad_x") + first),
                   self.gx.ptr, self.w.ptr, self.gz.ptr)

    def grad_y(self):
        first = "" if EAGER_ZERO else "_overwrite"
        self._call(getattr(self.lib, ("d8_deconv2d_grad_y" if self.deconv else "d8_conv2d_grad_y") + first),
                   self.x.ptr, self.gw.ptr, self.gz.ptr)

    def grad_xy(self):
        """both gradients from one call (d8_conv2d_grad_xy / d8_deconv2d_grad_xy), as this build's Conv2d / DeConv2d
        nodes issue them; on a layer whose products each leave compute units idle they share a launch"""
        from deep8_amd.capi import check
        B, IH, IW, IC = self.xd
        OC, FH, FW, _ = self.wd
        fn = self.lib.d8_deconv2d_grad_xy if self.deconv else self.lib.d8_conv2d_grad_xy
        if self.explicit:
            os.environ["D8_CONV_EXPLICIT"] = "1"
        try:
            check(fn(self.dt, self.x.ptr, self.gx.ptr, B, IH, IW, IC, self.w.ptr, self.gw.ptr, OC, FH, FW, self.gz.ptr, *self.geo,
                     0 if EAGER_ZERO else 3, self.ws.ptr, self.ws_bytes, self.stream))
        finally:
            if self.explicit:
                os.environ.pop("D8_CONV_EXPLICIT", None)

    def step(self):
        """forward + both gradients as the executor issues them: its zeroGradient() is deferred, so the
        first (here: only) product into each gradient is the overwrite form; --eager-zero fills and
        accumulates instead"""
        self.fwd()
        if EAGER_ZERO:
            self.gx.zero_()
            self.gw.zero_()
        self.grad_xy()

    def parts(self):
        f = self.flops / 3
        return {"fwd": (self.fwd, f), "grad_xy": (self.grad_xy, 2 * f), "grad_x": (self.grad_x, f), "grad_y": (self.grad_y, f)}

    def gemm_roofline(self, reps):
        """The pass-forward GEMM launch, timed alone with HIP events, against the MFMA peak of its
        element type.  Conv2d forward runs the tiled kernel (its tile loader reads the patch matrix
        straight from the image) over the rows that fill whole rounds of the chip and, in the same launch,
        over the remaining band of rows with the reduction split, then the band's reduction: both are
        inside the timed call; DeConv2d forward's GEMM (one product per filter tap,
        a single batched launch) is issued here through d8_gemm with the operator's own arguments."""
        from deep8_amd import capi
        B, IH, IW, IC = self.xd
        OC, FH, FW, _ = self.wd
        es = self.dtype.itemsize
        dtype = "f16" if self.dtype == np.float16 else "f32"
        flops = self.flops / 3
        q = self.lib.d8_deconv2d_scratch_bytes
        if self.deconv and q(self.dt, 0, B, IH, IW, IC, OC, FH, FW, *self.geo) == 0:
            fn = self.fwd  # no interim matrix: the whole forward is one launch
            name = ("gemm_tiled_kernel<%s> (DeConv2d forward: one launch over the %d residue classes of output pixels, "
                    "patch rows read from x by the tile loader)" % (dtype, self.geo[1] * self.geo[2]))
        elif self.deconv:
            T, M = FH * FW, B * IH * IW
            mat = capi.DeviceArray((M * T * OC,), self.dtype)
            fn = lambda: capi.check(self.lib.d8_gemm(self.dt, 0, 1, M, OC, IC, self.x.ptr, IC, 0, self.w.ptr, T * IC, IC, 0.0,
                                                     mat.ptr, T * OC, OC, T, None, 0, None))
            name = "gemm_tiled_kernel<%s> (DeConv2d forward: %d per-tap products [%dx%d]x[%dx%d]^T, one launch)" % (dtype, T, M, IC, OC, IC)
        else:
            fn = self.fwd
            name = "gemm_tiled_kernel<%s> (Conv2d forward, patch matrix read by the tile loader: one launch over whole rounds and the split remainder band, + the band's reduction, timed together)" % dtype
        ms = _time_events(fn, reps)
        ach = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "kernel": name, "achieved": round(ach, 2), "peak": PEAK[dtype], "unit": "TFLOP/s",
                "frac": round(ach / PEAK[dtype], 4), "launch_us": round(ms * 1e3, 2), **_traffic_fields(self.key)}


class ConvBiasReluWorkload(ConvWorkload):
    """Configuration 4's layer as it sits in a network: Conv2d -> Add (per-channel bias) -> ReLu, forward and backward.
    fused:   d8_conv2d_bias_relu | d8_bias_relu_grad, d8_conv2d_grad_xy                           (3 calls)
    unfused: d8_conv2d, d8_add, d8_relu | d8_relu_grad, d8_add_grad, d8_conv2d_grad_x, d8_conv2d_grad_y   (7 calls, the
             reference's sequence: deep8/src/math/Add.cu:21-52, ReLu.cu:20-116)"""

    def __init__(self, name, dtype, B, IH, IW, IC, OC, FH, FW, seed, fused):
        import ctypes
        from deep8_amd import capi
        ConvWorkload.__init__(self, name, dtype, False, B, IH, IW, IC, OC, FH, FW, True, 1, 1, seed)
        self.fused = fused
        r = np.random.default_rng(seed + 100)
        self.bias = _dev(r.standard_normal((OC,)).astype(np.float32).astype(dtype))
        zs = self.z.shape
        self.pre, self.sum, self.dpre = capi.DeviceArray(zs, dtype), capi.DeviceArray(zs, dtype), capi.DeviceArray(zs, dtype)
        self.gb = capi.DeviceArray((OC,), dtype)
        self.rows, self.OC = int(np.prod(zs[:-1])), OC
        I5 = ctypes.c_int * 5
        self.zd, self.bd = I5(zs[0], 1, zs[1], zs[2], OC), I5(1, 1, 1, 1, OC)
        self.rs_bytes = max(self.lib.d8_add_grad_scratch_bytes(self.dt, self.bd, self.zd),
                            self.lib.d8_bias_relu_grad_scratch_bytes(self.dt, self.rows, OC))
        self.rs = capi.DeviceArray((max(self.rs_bytes, 16),), np.uint8)
        nz = self.rows * OC * self.dtype.itemsize
        self.bytes += 4 * nz if fused else 9 * nz   # fused: z written by the product anyway; r z, r dz, w dpre (+ dpre read by the products)

    def step(self):
        from deep8_amd.capi import check
        L, n = self.lib, self.rows * self.OC
        B, IH, IW, IC = self.xd
        OC, FH, FW, _ = self.wd
        if self.fused:
            check(L.d8_conv2d_bias_relu(self.dt, self.x.ptr, B, IH, IW, IC, self.w.ptr, OC, FH, FW, self.bias.ptr, 1, self.z.ptr,
                                        *self.geo, self.ws.ptr, self.ws_bytes, None))
            check(L.d8_bias_relu_grad(self.dt, self.z.ptr, self.gz.ptr, self.dpre.ptr, self.gb.ptr, self.rows, OC, 0,
                                      self.rs.ptr, self.rs_bytes, None))
        else:
            self._call(L.d8_conv2d, self.x.ptr, self.w.ptr, self.pre.ptr)
            check(L.d8_add(self.dt, self.pre.ptr, self.zd, self.bias.ptr, self.bd, self.sum.ptr, self.zd, None))
            check(L.d8_relu(self.dt, self.sum.ptr, self.z.ptr, n, None))
            check(L.d8_relu_grad_overwrite(self.dt, self.sum.ptr, self.dpre.ptr, self.gz.ptr, n, None))
            check(L.d8_add_grad_overwrite(self.dt, self.gb.ptr, self.bd, self.dpre.ptr, self.zd, self.rs.ptr, self.rs_bytes, None))
        if self.fused:  # both gradients from one call, as the fused node issues them
            check(L.d8_conv2d_grad_xy(self.dt, self.x.ptr, self.gx.ptr, B, IH, IW, IC, self.w.ptr, self.gw.ptr, OC, FH, FW, self.dpre.ptr,
                                      *self.geo, 3, self.ws.ptr, self.ws_bytes, None))
        else:
            self._call(L.d8_conv2d_grad_x_overwrite, self.gx.ptr, self.w.ptr, self.dpre.ptr)
            self._call(L.d8_conv2d_grad_y_overwrite, self.x.ptr, self.gw.ptr, self.dpre.ptr)


class DeconvLiteralWorkload:
    """Benchmark configuration 5 at its literal geometry (28 -> 56, PyTorch's ConvTranspose2d(k=4, s=2, p=1)), which
    Deep8's DeConv2d does not admit (deep8/src/nodes/DeConv2d.cpp:36-52 allows 58 or 55): the operators' explicit-geometry
    entry points d8_deconv2d_ex / _grad_x_ex / _grad_y_ex with OH = OW = 56, padTop = padLeft = 2 -- the same three
    launches as the operator at Deep8's own geometries (workload c5)."""

    def __init__(self, name, seed):
        from deep8_amd import capi
        self.name, self.dtype, self.key = name, np.dtype(np.float16), name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        B, IH, IC, OC, F, S, OH, P = 16, 28, 128, 64, 4, 2, 56, 2
        self.B = B
        self.shape = (B, IH, IH, IC)
        self.filt = (OC, F, F)
        self.geo = (OH, OH, P, P, S, S)
        h = lambda a: _dev(a.astype(np.float32).astype(np.float16))
        self.x = h(r.standard_normal((B, IH, IH, IC)))
        self.w = h(r.standard_normal((OC, F, F, IC)) * np.sqrt(2.0 / (F * F * IC)))
        self.dz = h(r.standard_normal((B, OH, OH, OC)))
        self.z = capi.DeviceArray((B, OH, OH, OC), np.float16)
        self.dx = capi.DeviceArray((B, IH, IH, IC), np.float16)
        self.dw = capi.DeviceArray((OC, F, F, IC), np.float16)
        self.ws_bytes = max(self.lib.d8_deconv2d_scratch_bytes_ex(self.dt, wch, *self.shape, *self.filt, OH, OH, P, P, S, S) for wch in range(4))
        self.ws = capi.DeviceArray((max(self.ws_bytes, 16),), np.uint8)
        M, N = B * IH * IH, OC * F * F
        self.flops = 3 * 2.0 * M * N * IC
        nx, nw, nz = M * IC, N * IC, B * OH * OH * OC
        self.bytes = 2 * ((nx + nw + nz) + (nz + nw + nx) + (nx + nz + nw))  # overwrite forms: each pass reads two tensors, writes one

    def fwd(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv2d_ex(self.dt, self.x.ptr, *self.shape, self.w.ptr, *self.filt, self.z.ptr, *self.geo,
                                      self.ws.ptr, self.ws_bytes, None))

    def grad_x(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv2d_grad_x_ex(self.dt, self.dx.ptr, *self.shape, self.w.ptr, *self.filt, self.dz.ptr, *self.geo,
                                             0 if EAGER_ZERO else 1, self.ws.ptr, self.ws_bytes, None))

    def grad_y(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv2d_grad_y_ex(self.dt, self.x.ptr, *self.shape, self.dw.ptr, *self.filt, self.dz.ptr, *self.geo,
                                             0 if EAGER_ZERO else 1, self.ws.ptr, self.ws_bytes, None))

    def grad_xy(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv2d_grad_xy_ex(self.dt, self.x.ptr, self.dx.ptr, *self.shape, self.w.ptr, self.dw.ptr, *self.filt, self.dz.ptr,
                                              *self.geo, 0 if EAGER_ZERO else 3, self.ws.ptr, self.ws_bytes, None))

    def step(self):
        self.fwd()
        if EAGER_ZERO:
            self.dx.zero_()
            self.dw.zero_()
        self.grad_xy()

    kernel = "gemm_tiled_kernel<f16> (one launch for forward, one for dX and dW together; patch rows read by the tile loader)"

    def parts(self):
        f = self.flops / 3
        return {"fwd": (self.fwd, f), "grad_xy": (self.grad_xy, 2 * f), "grad_x": (self.grad_x, f), "grad_y": (self.grad_y, f)}


class GatherMapsWorkload:
    """d8_im2col and d8_col2im alone at config 4's size (fp32 B32 56x56x64, 3x3, stride 1, pad 1): the
    gather / scatter kernels of the reference's Conv2d lowering (deep8/src/math/Conv2d.cu:10-61, 64-118).
    HBM-bound: im2col reads the image and writes the patch matrix once; col2im reads the patch matrix once and
    read-modify-writes the image gradient."""

    def __init__(self, name, dtype, B, H, W, C, F, seed):
        from deep8_amd import capi
        self.name, self.dtype, self.key = name, np.dtype(dtype), name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        self.B = B
        self.geo = (B, H, W, C, H, W, F, F, 1, 1, 1, 1, F // 2, F // 2)
        self.x = _dev(r.standard_normal((B, H, W, C)).astype(np.float32).astype(dtype))
        self.col = capi.DeviceArray((B * H * W, F * F * C), dtype)
        self.gx = capi.DeviceArray((B, H, W, C), dtype, zero=True)
        es = self.dtype.itemsize
        self.im_bytes, self.col_bytes = es * B * H * W * C, es * B * H * W * F * F * C
        self.flops = float(B * H * W * F * F * C)  # the additions of col2im
        self.bytes = (self.im_bytes + self.col_bytes) + (self.col_bytes + 2 * self.im_bytes)

    def im2col(self):
        from deep8_amd.capi import check
        check(self.lib.d8_im2col(self.dt, self.x.ptr, self.col.ptr, *self.geo, None))

    def col2im(self):
        from deep8_amd.capi import check
        check(self.lib.d8_col2im(self.dt, self.col.ptr, self.gx.ptr, *self.geo, None))

    def step(self):
        self.im2col()
        self.col2im()

    def parts(self):
        """name -> (call, algorithmic bytes)"""
        return {"im2col": (self.im2col, self.im_bytes + self.col_bytes), "col2im": (self.col2im, self.col_bytes + 2 * self.im_bytes)}


class DeconvMapsWorkload:
    """d8_deconv_col2im and d8_deconv_im2col alone at configuration 5's literal size (half, B16 28x28 -> 56x56x64, 4x4,
    stride 2, pads 2): the gather maps of the reference's DeConv2d lowering in the reference's own matrix layout
    (deep8/src/math/DeConv2d.cu:11-58, 310-351).  HBM-bound: each reads or writes the 25.7 MB matrix once."""

    def __init__(self, name, seed):
        from deep8_amd import capi
        self.name, self.dtype, self.key = name, np.dtype(np.float16), name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        B, IH, OC, F, S, OH, P = 16, 28, 64, 4, 2, 56, 2
        self.B, self.geo = B, (B, IH, IH, OH, OH, OC, F, F, S, S, P, P)
        self.dz = _dev(r.standard_normal((B, OH, OH, OC)).astype(np.float32).astype(np.float16))
        self.mat = capi.DeviceArray((B * IH * IH, OC * F * F), np.float16, zero=True)
        self.z = capi.DeviceArray((B, OH, OH, OC), np.float16)
        self.mat_bytes, self.im_bytes = 2 * B * IH * IH * OC * F * F, 2 * B * OH * OH * OC
        self.flops = float(B * IH * IH * OC * F * F)
        self.bytes = 2 * (self.mat_bytes + self.im_bytes)

    def im2col(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv_im2col(self.dt, self.dz.ptr, self.mat.ptr, *self.geo, None))

    def col2im(self):
        from deep8_amd.capi import check
        check(self.lib.d8_deconv_col2im(self.dt, self.mat.ptr, self.z.ptr, *self.geo, None))

    def step(self):
        self.im2col()
        self.col2im()

    def parts(self):
        """name -> (call, algorithmic bytes)"""
        return {"deconv_im2col": (self.im2col, self.mat_bytes + self.im_bytes), "deconv_col2im": (self.col2im, self.mat_bytes + self.im_bytes)}


class BiasReluWorkload:
    """The element-wise steps after a convolution: Add (per-channel bias, broadcast) -> ReLu, and back:
    ReLuGrad -> AddGradY (bias gradient: a sum over batch, rows and columns).  HBM-bound."""

    def __init__(self, name, dtype, B, H, W, C, seed):
        import ctypes
        from deep8_amd import capi
        self.name, self.dtype, self.key = name, np.dtype(dtype), name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        self.n = B * H * W * C
        self.B = B
        self.z = _dev(r.standard_normal((B, H, W, C)).astype(np.float32).astype(dtype))
        self.b = _dev(r.standard_normal((1, C)).astype(np.float32).astype(dtype))
        self.gy = _dev(r.standard_normal((B, H, W, C)).astype(np.float32).astype(dtype))
        self.pre, self.act, self.gpre = (capi.DeviceArray((B, H, W, C), dtype) for _ in range(3))
        self.gb = capi.DeviceArray((1, C), dtype)
        I5 = ctypes.c_int * 5
        self.zd, self.bd = I5(B, 1, H, W, C), I5(1, 1, 1, 1, C)
        self.ws_bytes = self.lib.d8_add_grad_scratch_bytes(self.dt, self.bd, self.zd)
        self.ws = capi.DeviceArray((max(self.ws_bytes, 16),), np.uint8)
        es = self.dtype.itemsize
        self.flops = 4.0 * self.n
        # add: r z, w pre | relu: r pre, w act | relu_grad: r pre, r gy, w gpre (+ fill and read-back of gpre
        # with --eager-zero) | bias grad: r gpre
        self.bytes = es * self.n * (10 if EAGER_ZERO else 8)

    def add(self):
        from deep8_amd.capi import check
        check(self.lib.d8_add(self.dt, self.z.ptr, self.zd, self.b.ptr, self.bd, self.pre.ptr, self.zd, None))

    def relu(self):
        from deep8_amd.capi import check
        check(self.lib.d8_relu(self.dt, self.pre.ptr, self.act.ptr, self.n, None))

    def relu_grad(self):
        from deep8_amd.capi import check
        L = self.lib
        if EAGER_ZERO:
            self.gpre.zero_()
            check(L.d8_relu_grad(self.dt, self.pre.ptr, self.gpre.ptr, self.gy.ptr, self.n, None))
        else:  # a gradient whose zero fill is still pending is written, not added to
            check(L.d8_relu_grad_overwrite(self.dt, self.pre.ptr, self.gpre.ptr, self.gy.ptr, self.n, None))

    def bias_grad(self):
        from deep8_amd.capi import check
        L = self.lib
        if EAGER_ZERO:
            self.gb.zero_()
            check(L.d8_add_grad(self.dt, self.gb.ptr, self.bd, self.gpre.ptr, self.zd, self.ws.ptr, self.ws_bytes, None))
        else:
            check(L.d8_add_grad_overwrite(self.dt, self.gb.ptr, self.bd, self.gpre.ptr, self.zd, self.ws.ptr, self.ws_bytes, None))

    def step(self):
        self.add()
        self.relu()
        self.relu_grad()
        self.bias_grad()

    def parts(self):
        """name -> (call, algorithmic bytes): what each kernel must read and write once"""
        nb = self.dtype.itemsize * self.n
        return {"add (bias broadcast)": (self.add, 2 * nb), "relu": (self.relu, 2 * nb),
                "relu_grad": (self.relu_grad, (5 if EAGER_ZERO else 3) * nb), "bias_grad (sum over rows)": (self.bias_grad, nb)}


class PoolWorkload:
    """MaxPooling2d 2x2 / 2 forward and gradient on config 4's activations.  HBM-bound gathers."""

    def __init__(self, name, dtype, B, H, W, C, seed):
        from deep8_amd import capi
        self.name, self.dtype, self.key = name, np.dtype(dtype), name.split(":")[0]
        self.lib = capi.init()
        self.dt = capi.dtype_id(self.dtype)
        r = np.random.default_rng(seed)
        self.B, self.dims = B, (B, H, W, C)
        self.x = _dev(r.standard_normal((B, H, W, C)).astype(np.float32).astype(dtype))
        self.y = capi.DeviceArray((B, H // 2, W // 2, C), dtype)
        self.gy = _dev(r.standard_normal((B, H // 2, W // 2, C)).astype(np.float32).astype(dtype))
        self.gx = capi.DeviceArray((B, H, W, C), dtype)
        n, es = B * H * W * C, self.dtype.itemsize
        self.flops = 2.0 * n
        # forward: r x, w y | gradient: r x, r gy, w gx (+ fill and read-back of gx with --eager-zero)
        self.bytes = es * (n + n // 4 + n + n // 4 + n + (2 * n if EAGER_ZERO else 0))

    def fwd(self):
        from deep8_amd.capi import check
        check(self.lib.d8_maxpool2d(self.dt, self.x.ptr, self.y.ptr, *self.dims, 2, 2, 0, 2, 2, None))

    def grad(self):
        from deep8_amd.capi import check
        if EAGER_ZERO:
            self.gx.zero_()
            check(self.lib.d8_maxpool2d_grad(self.dt, self.x.ptr, self.gx.ptr, self.gy.ptr, *self.dims, 2, 2, 0, 2, 2, None))
        else:
            check(self.lib.d8_maxpool2d_grad_overwrite(self.dt, self.x.ptr, self.gx.ptr, self.gy.ptr, *self.dims, 2, 2, 0, 2, 2, None))

    def step(self):
        self.fwd()
        self.grad()

    def parts(self):
        """name -> (call, algorithmic bytes)"""
        nb = self.dtype.itemsize * int(np.prod(self.dims))
        return {"maxpool2d": (self.fwd, nb + nb // 4), "maxpool2d_grad": (self.grad, nb + nb // 4 + nb + (2 * nb if EAGER_ZERO else 0))}


def _uni(r, s):
    return r.uniform(-1, 1, s).astype(np.float32)


ZERO_OPERANDS = False   # --operands zeros: same launches on all-zero data (shows how much of the rate the data costs)


def make_workload(key):
    U = {"x": _uni, "y": _uni, "dz": _uni}
    if ZERO_OPERANDS:
        zero = lambda r, s: np.zeros(s, np.float32)
        U = {"x": zero, "y": zero, "dz": zero}
    if key == "c1":
        return MatMulWorkload("c1: MatrixMultiply fwd+dX+dY fp32 [64x128]x[128x256]", np.float32,
                              (1, 64, 128), (1, 128, 256), U, 1)
    if key == "c2a":
        return MatMulWorkload("c2a: MatrixMultiply fwd+dX+dY fp32 batch 32 of [512x512]x[512x512]", np.float32,
                              (32, 512, 512), (32, 512, 512), U, 2)
    if key == "c2b":
        return MatMulWorkload("c2b: MatrixMultiply fwd+dX+dY fp32 A batch 32 [512x512], B batch 1 (shared)",
                              np.float32, (32, 512, 512), (1, 512, 512), U, 3)
    if key in ("f1", "f1s"):  # a fully connected layer: x [1024 x 1024] . W [1024 x 1024], half / fp32
        g = {"x": lambda r, s: r.standard_normal(s).astype(np.float32),
             "y": lambda r, s: (r.standard_normal(s) / 32.0).astype(np.float32),
             "dz": lambda r, s: r.standard_normal(s).astype(np.float32)}
        return MatMulWorkload("%s: MatrixMultiply fwd+dX+dY %s [1024x1024]x[1024x1024] (a fully connected layer: both gradients "
                              "in one launch of the tiled kernel)" % (key, "half" if key == "f1" else "fp32"),
                              np.float16 if key == "f1" else np.float32, (1, 1024, 1024), (1, 1024, 1024), g, 13)
    if key == "c3":
        g = {"x": lambda r, s: (r.standard_normal(s) / 64.0).astype(np.float32),
             "y": lambda r, s: (r.standard_normal(s) / 64.0).astype(np.float32),
             "dz": lambda r, s: r.standard_normal(s).astype(np.float32)}
        return MatMulWorkload("c3: MatrixMultiply fwd+dX+dY half [4096x4096]x[4096x4096]", np.float16,
                              (1, 4096, 4096), (1, 4096, 4096), U if ZERO_OPERANDS else g, 4)
    if key == "c4":
        return ConvWorkload("c4: Conv2d fwd+dX+dW fp32 B32 56x56x64 3x3x64->64 s1 same", np.float32, False,
                            32, 56, 56, 64, 64, 3, 3, True, 1, 1, 5)
    if key == "c4h":
        return ConvWorkload("c4h: Conv2d fwd+dX+dW half B32 56x56x64 3x3x64->64 s1 same (configuration 4's layer in half precision)",
                            np.float16, False, 32, 56, 56, 64, 64, 3, 3, True, 1, 1, 5)
    if key == "c4x":
        return ConvWorkload("c4x: Conv2d fwd+dX+dW fp32 B32 56x56x64 3x3x64->64 s1 same, the reference's lowering "
                            "(im2col -> GEMM, GEMM -> col2im, 231 MB interim matrix)", np.float32, False,
                            32, 56, 56, 64, 64, 3, 3, True, 1, 1, 5, explicit=True)
    if key in ("c4e", "c4e_unfused"):
        return ConvBiasReluWorkload("%s: Conv2d + bias Add + ReLu fwd+bwd fp32 B32 56x56x64 3x3x64->64, %s" % (
            key, "bias and ReLu in the product's store, ReLuGrad + bias gradient in one pass" if key == "c4e" else
            "every operator a call of its own (the reference's sequence)"), np.float32, 32, 56, 56, 64, 64, 3, 3, 5, key == "c4e")
    if key == "i4":
        return GatherMapsWorkload("i4: d8_im2col + d8_col2im alone at config 4's size, fp32 B32 56x56x64 3x3 s1 pad 1",
                                  np.float32, 32, 56, 56, 64, 3, 11)
    if key == "k5":
        return DeconvMapsWorkload("k5: d8_deconv_im2col + d8_deconv_col2im alone at config 5's literal size, half B16 28x28 -> 56x56x64 4x4 s2", 12)
    if key == "c5":
        return ConvWorkload("c5: DeConv2d fwd+dX+dW half B16 28x28x128 4x4 s2 -> 58x58x64 (Deep8 covered=false)",
                            np.float16, True, 16, 28, 28, 128, 64, 4, 4, False, 2, 2, 6)
    if key == "c5l":
        return DeconvLiteralWorkload("c5l: DeConv2d fwd+dX+dW half B16 28x28x128 4x4 s2 -> 56x56x64 (configuration 5 as written, "
                                     "through the explicit-geometry operator entry points)", 9)
    if key == "d3":
        return MatMulWorkload("d3: MatrixMultiply fwd+dX+dY double [2048x2048]x[2048x2048]", np.float64,
                              (1, 2048, 2048), (1, 2048, 2048), U, 10)
    if key == "e4":
        return BiasReluWorkload("e4: bias Add + ReLu fwd+bwd on config 4's output, fp32 B32 56x56x64", np.float32, 32, 56, 56, 64, 7)
    if key == "p4":
        return PoolWorkload("p4: MaxPooling2d 2x2/2 fwd+bwd on config 4's output, fp32 B32 56x56x64", np.float32, 32, 56, 56, 64, 8)
    raise SystemExit("unknown workload %r" % key)


def _repeat_for(fn, seconds):
    """run fn (after one untimed call) until about `seconds` have passed; returns (calls, elapsed)"""
    fn()
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= seconds:
            return n, dt


def cpu_baseline(key, seconds=12.0):
    """Deep8's CPU path on a bounded sample of the workload (forward + both gradients), repeated
    for about `seconds` of CPU work."""
    import oracle
    src = oracle.ref if oracle.ref is not None else oracle.port
    kind = "reference" if oracle.ref is not None else "port"
    r = np.random.default_rng(9)
    if key in ("e4", "p4"):
        # element-wise and pooling operators run on the CPU device's Eigen thread pool in the reference
        B = 8
        x = r.standard_normal((B, 56, 56, 64)).astype(np.float32)
        if key == "e4":
            b, gy = r.standard_normal((1, 64)).astype(np.float32), r.standard_normal(x.shape).astype(np.float32)

            def one():
                pre = src.add(x, b)
                src.relu(pre)
                gpre = src.relu_grad(pre, gy)
                src.add_grad(1, x, b, gpre) if kind == "reference" else src.add_grad(b, gpre)
        else:
            gy = r.standard_normal((B, 28, 28, 64)).astype(np.float32)

            def one():
                src.pool2d(True, x, 2, 2, False, 2, 2)
                src.pool2d_grad(True, x, gy, 2, 2, False, 2, 2)
        n, dt = _repeat_for(one, seconds)
        return {"value": n * B / dt, "unit": "images/s", "cores": src.threads(), "kind": kind,
                "sample": "%s fwd+bwd on %d images x %d repeats (fp32 CPU path, host-side array copies included), %.1f s"
                          % (key, B, n, dt)}
    if key == "k5":
        port = oracle.port
        B = 4
        dz = r.standard_normal((B, 56, 56, 64)).astype(np.float32)

        def one():
            m = port.deconv_im2col(dz, 28, 28, 4, 4, 2, 2, 2, 2)
            port.deconv_col2im(m, B, 28, 28, 56, 56, 64, 4, 4, 2, 2, 2, 2)
        n, dt = _repeat_for(one, seconds)
        return {"value": n * B / dt, "unit": "images/s", "cores": port.threads(), "kind": "port",
                "sample": "deconv_im2col + deconv_col2im on %d images x %d repeats (fp32, C restatement), %.1f s" % (B, n, dt)}
    if key == "i4":
        # the reference's CPU path never materialises the patch matrix (it is a lazy Eigen expression), so the
        # two maps are timed on the C restatement of the reference's GPU kernels' index maps
        port = oracle.port
        B = 8
        x = r.standard_normal((B, 56, 56, 64)).astype(np.float32)
        gx = np.zeros_like(x)

        def one():
            col = port.im2col(x, 56, 56, 3, 3, 1, 1, 1, 1, 1, 1)
            port.col2im(col, gx, 56, 56, 3, 3, 1, 1, 1, 1, 1, 1)
        n, dt = _repeat_for(one, seconds)
        return {"value": n * B / dt, "unit": "images/s", "cores": port.threads(), "kind": "port",
                "sample": "im2col + col2im on %d images x %d repeats (fp32, C restatement), %.1f s" % (B, n, dt)}
    if key in ("c4", "c4h", "c4x", "c4e", "c4e_unfused", "c5"):
        # the reference runs Conv2d/DeConv2d on Eigen's thread pool: all host cores
        B = 8
        if key != "c5":
            x, w = r.standard_normal((B, 56, 56, 64)).astype(np.float32), r.standard_normal((64, 3, 3, 64)).astype(np.float32)
            args, f3 = (True, 1, 1, 1, 1), (src.conv2d, src.conv2d_grad_x, src.conv2d_grad_y)
        else:
            x, w = r.standard_normal((B, 28, 28, 128)).astype(np.float32), r.standard_normal((64, 4, 4, 128)).astype(np.float32)
            args, f3 = (False, 2, 2), (src.deconv2d, src.deconv2d_grad_x, src.deconv2d_grad_y)
        gz = r.standard_normal(f3[0](x, w, *args).shape).astype(np.float32)

        def one():
            f3[0](x, w, *args)
            f3[1](x, w, gz, *args)
            f3[2](x, w, gz, *args)
        n, dt = _repeat_for(one, seconds)
        return {"value": n * B / dt, "unit": "images/s", "cores": src.threads(), "kind": kind,
                "sample": "%s fwd+dX+dW on %d images x %d repeats (fp32 CPU path), %.1f s" % (key, B, n, dt)}
    # MatrixMultiply: Eigen's dense product is single-threaded in the reference build
    wide = np.float64 if key == "d3" else np.float32
    if key == "d3":
        m, k, n_, b = 256, 2048, 2048, 1
    elif key == "c3":
        m, k, n_, b = 256, 4096, 4096, 1
    elif key in ("c2a", "c2b"):
        m, k, n_, b = 512, 512, 512, 8
    else:
        m, k, n_, b = 64, 128, 256, 1
    x, y = r.uniform(-1, 1, (b, m, k)).astype(wide), r.uniform(-1, 1, (1 if key != "c2a" else b, k, n_)).astype(wide)
    dz = r.uniform(-1, 1, (b, m, n_)).astype(wide)

    def one():
        src.matmul(x, y)
        src.matmul_grad_x(x, y, dz)
        src.matmul_grad_y(x, y, dz)
    if key == "d3":
        with oracle.float64():
            n, dt = _repeat_for(one, seconds)
    else:
        n, dt = _repeat_for(one, seconds)
    flops = n * 3 * 2.0 * b * m * k * n_
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1 if kind == "reference" else src.threads(),
            "kind": kind,
            "sample": "fwd+dX+dY of %d x [%dx%d]x[%dx%d] %s x %d repeats, %.1f s"
                      % (b, m, k, k, n_, "fp64" if key == "d3" else "fp32 (the reference has no CPU half)", n, dt)}


def calibrate_copy(mib):
    """A plain copy of known size (the im2col kernel with a 1x1 filter is exactly that), run under
    `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` to find what those counters read per byte moved."""
    from deep8_amd import capi
    lib = capi.init()
    n = mib * (1 << 20) // 4
    rows = n // 64
    src = capi.DeviceArray((rows, 64), np.float32, zero=True)
    dst = capi.DeviceArray((rows, 64), np.float32, zero=True)
    for _ in range(5):
        capi.check(lib.d8_im2col(capi.FLOAT32, src.ptr, dst.ptr, 1, rows, 1, 64, rows, 1, 1, 1, 1, 1, 1, 1, 0, 0, None))
    capi.sync()
    print(json.dumps({"copy_kernel": "im2col_kernel (1x1 filter)", "bytes_read": rows * 256, "bytes_written": rows * 256}))


def graph_replay_ms(wl, steps, warmup):
    """ms per step of a MatrixMultiply workload whose step is captured once into a HIP graph (d8_graph_begin /
    d8_graph_end) and replayed: what a caller gets who removes the per-launch latency of a small product that way."""
    import ctypes
    from deep8_amd import capi
    lib = capi.init()
    capi.sync()
    side, graph = ctypes.c_void_p(), ctypes.c_void_p()
    capi.check(lib.d8_stream_create(ctypes.byref(side)))
    wl.stream = side
    try:
        for _ in range(3):
            wl.step()
        capi.sync(side)
        capi.check(lib.d8_graph_begin(side))
        wl.step()
        capi.check(lib.d8_graph_end(side, ctypes.byref(graph)))
        for _ in range(warmup):
            capi.check(lib.d8_graph_launch(graph, side))
        capi.sync(side)
        t = capi.Timer(side)
        t.start()
        for _ in range(steps):
            capi.check(lib.d8_graph_launch(graph, side))
        return t.stop_ms() / steps
    finally:
        wl.stream = None
        capi.sync(side)
        lib.d8_graph_destroy(graph)
        lib.d8_stream_destroy(side)


WIDE_DIAGNOSTICS = {"same_k": ["D8_DIAG_SAME_K"], "no_stores": ["D8_DIAG_NO_STORES"],
                    "no_fragment_reads": ["D8_DIAG_NO_FRAGMENT_READS"], "no_loads": ["D8_DIAG_NO_LOADS"],
                    "no_barrier": ["D8_DIAG_NO_BARRIER"],
                    "mfma_only": ["D8_DIAG_NO_FRAGMENT_READS", "D8_DIAG_NO_LOADS", "D8_DIAG_NO_BARRIER"]}


def build_wide_diagnostic(name):
    """compiles deep8_amd/csrc/diag/gemm_wide_diag.hip (the fp16 kernel with one of its parts left out) and links it,
    in place of gemm_wide.hip's object, with the library's other objects (deep8_amd/csrc/obj, left by
    __graft_entry__.build(); compiled here where absent) into a scratch library; returns its path"""
    import subprocess
    import tempfile
    import __graft_entry__ as ge
    csrc = os.path.join(ROOT, "deep8_amd", "csrc")
    tmp = tempfile.mkdtemp(prefix="d8_wide_diag_")
    obj, lib = os.path.join(tmp, "gemm_wide.o"), os.path.join(tmp, "libdeep8_hip_%s.so" % name)
    subprocess.check_call([ge.HIPCC] + ge.HIP_FLAGS + ["-D" + d for d in WIDE_DIAGNOSTICS[name]] +
                          ["-c", os.path.join(csrc, "diag", "gemm_wide_diag.hip"), "-o", obj], stderr=subprocess.DEVNULL)
    objs, jobs = [obj], []
    for src in sorted(f for f in os.listdir(csrc) if f.endswith(".hip") and f != "gemm_wide.hip"):
        have = os.path.join(csrc, "obj", src[:-4] + ".o")
        if os.path.exists(have):
            objs.append(have)
        else:
            o = os.path.join(tmp, src[:-4] + ".o")
            jobs.append(subprocess.Popen([ge.HIPCC] + ge.HIP_FLAGS + ["-c", os.path.join(csrc, src), "-o", o], stderr=subprocess.DEVNULL))
            objs.append(o)
    for j in jobs:
        if j.wait() != 0:
            raise SystemExit("bench.py: compiling the library's sources for the diagnostic build failed")
    subprocess.check_call([ge.HIPCC] + ge.HIP_FLAGS + ["-shared", "-o", lib] + objs, stderr=subprocess.DEVNULL)
    return lib


def phase_record(launches=12):
    """The fp16 4096^3 launches of workload c3 with the kernel's own phase record switched on (D8_GEMM_STAMPS):
    every workgroup notes the wall clock (100 MHz, common to the chip) at its start, after its prologue, after
    its K loop and after its last store was acknowledged, and the shader clock around the loop.  Prints, per
    product, the phases in microseconds and the shader clock per XCD (workgroup id mod 8).  A diagnostic: it
    shows how much of a launch is the loop and at which clock the loop runs on the config's data."""
    from deep8_amd import capi
    lib = capi.init()
    wl = make_workload("c3")
    n = 4096
    forms = (("forward NN", 0, 0, wl.x, wl.y), ("dX NT", 0, 1, wl.dz, wl.y), ("dY TN", 1, 0, wl.x, wl.dz))
    out = capi.DeviceArray((n, n), np.float16)
    recs = [capi.DeviceArray((256 * 6,), np.uint64, zero=True) for _ in range(launches)]
    for name, ta, tb, A, B in forms:
        def launch(i):
            capi.check(lib.d8_gemm(wl.dt, ta, tb, n, n, n, A.ptr, n, 0, B.ptr, n, 0, 0.0, out.ptr, n, 0, 1,
                                   recs[i].ptr, 256 * 6 * 8, None))
        _settle(lambda: launch(0))
        for i in range(launches):
            launch(i)
        capi.sync()
        t = capi.Timer(None)
        t.start()
        for i in range(launches):
            launch(i)
        ms = t.stop_ms() / launches
        d = [r.numpy().astype(np.int64).reshape(256, 6) for r in recs]
        if not d[-1][:, 3].all():
            raise SystemExit("no phase record was written: is D8_GEMM_STAMPS set and does the product take gemm_wide_kernel?")
        print("%s: %.1f us per launch by HIP events over %d launches (%.0f TFLOP/s)" % (name, ms * 1e3, launches, 2.0 * n**3 / ms / 1e9))
        r = d[-1]
        t0 = r[:, 0].min()
        us = lambda v: v / 100.0
        pro, loop, epi = us(r[:, 1] - r[:, 0]), us(r[:, 2] - r[:, 1]), us(r[:, 3] - r[:, 2])
        ghz = (r[:, 5] - r[:, 4]) / (loop * 1e3)
        gap = us(r[:, 0].min() - d[-2][:, 3].max())
        print("  last launch: prologue %.1f us, loop %.1f-%.1f (mean %.1f), epilogue until the last store is acknowledged "
              "%.1f-%.1f; last workgroup done %.1f us after the first started; %.1f us from the end of the previous launch "
              "to the first workgroup of this one" % (pro.mean(), loop.min(), loop.max(), loop.mean(), epi.min(), epi.max(),
                                                      us(r[:, 3].max() - t0), gap))
        print("  shader clock during the loop, per XCD: " + ", ".join(
            "%.2f" % ghz[np.arange(256) % 8 == x].mean() for x in range(8)) + " GHz; cycles per K step %.0f" % (
            (r[:, 5] - r[:, 4]).mean() / (n // 64)))
    pair_phase_record(wl, launches)


def pair_phase_record(wl, launches=12):
    """the same record for both gradients as ONE launch (d8_matmul_grad_xy): 256 workgroups, each a tile of dX and then
    a tile of dY; what separates the two K loops of a workgroup is printed as its turn-around"""
    from deep8_amd import capi
    lib = capi.init()
    n = 4096
    recs = [capi.DeviceArray((512 * 6,), np.uint64, zero=True) for _ in range(launches)]

    def launch(i):
        capi.check(lib.d8_matmul_grad_xy(wl.dt, wl.x.ptr, wl.dx.ptr, 1, n, n, wl.y.ptr, wl.dy.ptr, 1, n, n, wl.dz.ptr, 3,
                                         recs[i].ptr, 512 * 6 * 8, None))
    _settle(lambda: launch(0))
    for i in range(launches):
        launch(i)
    capi.sync()
    t = capi.Timer(None)
    t.start()
    for i in range(launches):
        launch(i)
    ms = t.stop_ms() / launches
    r = recs[-1].numpy().astype(np.int64).reshape(512, 6)
    if not r[:, 3].all():
        raise SystemExit("no phase record was written for the launch of two products")
    us = lambda v: v / 100.0
    first, second = r[:256], r[256:]
    print("dX NT + dY TN as one launch: %.1f us per launch by HIP events over %d launches (%.0f TFLOP/s)" % (
        ms * 1e3, launches, 4.0 * n**3 / ms / 1e9))
    for name, q in (("dX tiles", first), ("dY tiles", second)):
        loop = us(q[:, 2] - q[:, 1])
        ghz = (q[:, 5] - q[:, 4]) / (loop * 1e3)
        print("  %s: K loop %.1f-%.1f us (mean %.1f) at %.2f GHz, %.0f cycles per K step" % (
            name, loop.min(), loop.max(), loop.mean(), ghz.mean(), (q[:, 5] - q[:, 4]).mean() / (n // 64)))
    turn = us(second[:, 1] - first[:, 2])
    print("  prologue %.1f us; from the end of a workgroup's first K loop to the start of its second (the next tile's first "
          "loads issued, the epilogue, the wait for those loads) %.1f-%.1f us (mean %.1f); last epilogue until its stores "
          "are acknowledged %.1f-%.1f us; last workgroup done %.1f us after the first started" % (
              us(first[:, 1] - first[:, 0]).mean(), turn.min(), turn.max(), turn.mean(),
              us(second[:, 3] - second[:, 2]).min(), us(second[:, 3] - second[:, 2]).max(), us(r[:, 3].max() - r[:, 0].min())))


def tiled_phase_record(key, launches=8):
    """The calls of a workload that run gemm_tiled_kernel (the fp32 products, the convolutions) with the kernel's
    per-workgroup phase record switched on (d8_gemm_phase_record): for each part of the step, when its workgroups
    started, how long their prologue, K loop and epilogue took, at which shader clock the loop ran, how many tiles
    a CU worked on and when they ended, and the same for the workgroups of a remainder band riding in the launch.
    A diagnostic: it shows what a launch's time is made of (the matrix pipe's own share is printed beside it)."""
    from deep8_amd import capi
    lib = capi.init()
    wl = make_workload(key)
    nrec = 1 << 14
    bufs = [capi.DeviceArray((nrec * 8,), np.uint64, zero=True) for _ in range(launches)]
    peak_per_cu_cycle = {2: 2048.0, 4: 256.0}[wl.dtype.itemsize]  # flops per CU and cycle of the dense MFMA peak
    for name, (fn, flops) in wl.parts().items():
        capi.check(lib.d8_gemm_phase_record(None, 0))
        for b in bufs:  # (records of the previous part)
            b.zero_()
        _settle(fn)
        for b in bufs:  # (each launch writes its records from index 0: one buffer per launch)
            capi.check(lib.d8_gemm_phase_record(b.ptr, nrec * 64))
            fn()
        capi.sync()
        capi.check(lib.d8_gemm_phase_record(None, 0))
        r = bufs[-1].numpy().astype(np.int64).reshape(nrec, 8)
        r = r[r[:, 3] != 0]
        if not len(r):
            print("%s: no records (the call does not run gemm_tiled_kernel, or its grid exceeds %d workgroups)" % (name, nrec), flush=True)
            continue
        us = lambda v: v / 100.0
        t0 = r[:, 0].min()
        start, end = us(r[:, 0] - t0), us(r[:, 3] - t0)
        pro, loop, epi = us(r[:, 1] - r[:, 0]), us(r[:, 2] - r[:, 1]), us(r[:, 3] - r[:, 2])
        band = (r[:, 7] & 1) == 1
        second = (r[:, 7] >> 1) == 1  # a launch of two products: the workgroups of the second (the gradient of x)
        key_cu = ((r[:, 6] >> 32) & 0xf) * 65536 + (r[:, 6] & 0xff00)  # XCD, and the SE / SH / CU bits of HW_ID
        cus = len(np.unique(key_cu))
        ghz = ((r[:, 5] - r[:, 4]) / np.maximum(loop * 1e3, 1e-9))[~band].mean()
        pipe_us = flops / (cus * peak_per_cu_cycle * ghz * 1e9) * 1e6
        print("%s: %d workgroups on %d CUs (%d of them on the remainder band); first start to last store acknowledged "
              "%.1f us; the matrix pipe alone at the loop's own clock (%.2f GHz) would need %.1f us" % (
                  name, len(r), cus, band.sum(), end.max(), ghz, pipe_us), flush=True)
        groups = ((("tiles", ~band), ("band pieces", band)) if not second.any() else
                  (("filter-gradient pieces", ~second), ("input-gradient tiles", second)))
        for label, m in groups:
            if not m.any():
                continue
            print("  %s: start %.1f-%.1f us; prologue %.1f-%.1f (mean %.1f); K loop %.1f-%.1f (mean %.1f); epilogue "
                  "%.1f-%.1f (mean %.1f); end %.1f-%.1f" % (label, start[m].min(), start[m].max(), pro[m].min(), pro[m].max(),
                                                          pro[m].mean(), loop[m].min(), loop[m].max(), loop[m].mean(),
                                                          epi[m].min(), epi[m].max(), epi[m].mean(), end[m].min(), end[m].max()))
        _, per_cu = np.unique(key_cu[~band], return_counts=True)
        print("  tiles per CU: " + ", ".join("%d CUs x %d" % (c, n) for n, c in zip(*np.unique(per_cu, return_counts=True))))
        edges = np.arange(0, min(end.max(), 1000.0) + 5, 5)
        hist, _ = np.histogram(end[~band], bins=edges)
        print("  tiles ending in each 5 us: " + " ".join("%d" % h for h in hist))
        one = np.where(key_cu == key_cu[np.argmin(start)])[0]
        print("  one CU: " + "; ".join("%s start %.1f prologue %.1f loop %.1f epilogue %.1f end %.1f" % (
            "band piece" if band[i] else "tile", start[i], pro[i], loop[i], epi[i], end[i]) for i in one[np.argsort(start[one])]))


def main():
    global ZERO_OPERANDS, EAGER_ZERO, SETTLE_MS, REPS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-others", action="store_true")
    ap.add_argument("--operands", choices=("config", "zeros"), default="config",
                    help="zeros: run the MatrixMultiply workloads on all-zero operands (a diagnostic: the chip "
                         "clocks higher when the data does not toggle; not a valid benchmark value)")
    ap.add_argument("--eager-zero", action="store_true",
                    help="zero-fill the gradients and accumulate (the reference's literal "
                         "sequence) instead of the executor's deferred zeroing + overwrite")
    ap.add_argument("--reps", type=int, default=REPS,
                    help="repetitions of the timed region of --steps steps; ms_per_step is their median")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed work issued before every measurement so that it runs at the sustained clock "
                         "(0: start from an idle device)")
    ap.add_argument("--phases", action="store_true",
                    help="only print the kernels' own phase record: of workload c3's three products (see phase_record), or, with "
                         "--workload, of another workload's tiled launches (see tiled_phase_record)")
    ap.add_argument("--wide-diagnostic", choices=sorted(WIDE_DIAGNOSTICS), default=None,
                    help="with --phases: compile the fp16 kernel with one of its diagnostic switches into a scratch "
                         "library and print that build's phase record (see the header of deep8_amd/csrc/gemm_wide.hip)")
    ap.add_argument("--step-only", action="store_true",
                    help="time the steps and print a short line: nothing else is launched (no per-call timings, no "
                         "second sequence, no CPU baseline), so that a kernel trace of the run holds the step's kernels only")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="only run a plain copy of this size (counter calibration under rocprofv3 --pmc)")
    a = ap.parse_args()
    SETTLE_MS = a.settle_ms
    REPS = max(1, a.reps)
    ZERO_OPERANDS = a.operands == "zeros"
    EAGER_ZERO = a.eager_zero
    if a.gpus != 1:
        raise SystemExit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no collectives, "
                         "no second device anywhere in the path)" % a.gpus)

    if a.phases:
        os.environ["D8_GEMM_STAMPS"] = "1"  # read by the library at its first launch
    from deep8_amd import capi
    if a.wide_diagnostic:
        if not a.phases:
            raise SystemExit("--wide-diagnostic goes with --phases")
        capi.LIB_PATH = build_wide_diagnostic(a.wide_diagnostic)
        print("diagnostic build of gemm_wide.hip: " + " ".join("-D" + d for d in WIDE_DIAGNOSTICS[a.wide_diagnostic]), flush=True)
    capi.init()
    if a.calibrate_copy:
        return calibrate_copy(a.calibrate_copy)
    if a.phases:
        return phase_record() if a.workload == "c3" else tiled_phase_record(a.workload)

    wl = make_workload(a.workload)
    ms, samples = _time_steps(wl.step, a.steps, a.warmup)
    dtype = {2: "f16", 4: "f32", 8: "f64"}[wl.dtype.itemsize]
    if a.step_only:
        print(json.dumps({"workload": wl.name + (", fill + accumulate" if EAGER_ZERO else ""), "steps": a.steps, "warmup": a.warmup,
                          "settle_ms": SETTLE_MS, "ms_per_step": round(ms, 4), "ms_per_step_samples": [round(v, 4) for v in samples],
                          "tflops": round(wl.flops / (ms * 1e-3) / 1e12, 2), "dtype": dtype}), flush=True)
        return
    is_conv = isinstance(wl, ConvWorkload)
    is_mm = isinstance(wl, MatMulWorkload)
    is_stream = isinstance(wl, (BiasReluWorkload, PoolWorkload, GatherMapsWorkload, DeconvMapsWorkload))  # HBM-bound kernels
    tflops = wl.flops / (ms * 1e-3) / 1e12

    def time_parts(table):
        res = {}
        for pname, (fn, amount) in table.items():
            pms = _time_events(fn, max(200, a.steps) if is_stream else max(5, a.steps))  # 10 us kernels: more launches per timing
            if is_stream:
                res[pname] = {"ms": round(pms, 4), "algorithmic_GBps": round(amount / (pms * 1e-3) / 1e9, 1)}
            else:
                res[pname] = {"ms": round(pms, 4), "tflops": round(amount / (pms * 1e-3) / 1e12, 2)}
        return res

    parts = time_parts(wl.parts())
    eager = None
    if is_conv:
        roof = wl.gemm_roofline(max(5, a.steps))
    elif is_stream:
        # the kernel the step spends most of its time in, against the HBM peak: the bytes it must read
        # and write once / its duration alone (HIP events on the launch stream)
        pname = max(parts, key=lambda k: parts[k]["ms"])
        ach = parts[pname]["algorithmic_GBps"]
        roof = {"bound": "hbm", "kernel": pname, "achieved": ach, "peak": HBM_PEAK, "unit": "GB/s",
                "frac": round(ach / HBM_PEAK, 4), "launch_us": round(parts[pname]["ms"] * 1e3, 2),
                **_traffic_fields(a.workload, pname)}
        for k, v in parts.items():  # every kernel of the step against the HBM peak
            v["frac_of_hbm_peak"] = round(v["algorithmic_GBps"] / HBM_PEAK, 4)
    else:
        # a MatrixMultiply step is the forward call and the call for both gradients (one launch of the large-output
        # fp16 kernel each; one launch per product elsewhere): flops per product / duration per product of those
        # calls, HIP events on the launch stream
        avg_ms = ((parts["fwd"]["ms"] + parts["grad_xy"]["ms"]) / 3 if "grad_xy" in parts else
                  sum(p["ms"] for p in parts.values()) / len(parts))
        ach = wl.flops / 3 / (avg_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "kernel": wl.kernel, "achieved": round(ach, 2), "peak": PEAK[dtype],
                "unit": "TFLOP/s", "frac": round(ach / PEAK[dtype], 4), "launch_us": round(avg_ms * 1e3, 2),
                **_traffic_fields(a.workload)}
        roof["mfma_stream_ceiling"] = mfma_stream_ceiling(wl, dtype)
        if is_mm and not EAGER_ZERO:
            # the reference executor's literal sequence beside the deferred-zeroing one `value` is quoted on:
            # forward, fill both gradients, two beta = 1 products (same flops, same result)
            ems, esamples = _time_steps(wl.step_eager_zero, a.steps, a.warmup)
            acc = time_parts(wl.parts_accumulate())
            parts.update(acc)
            eavg = (parts["fwd"]["ms"] + acc["grad_xy_accumulate"]["ms"]) / 3
            et = wl.flops / (ems * 1e-3) / 1e12
            eager = {"sequence": "forward, zero-fill dX and dY, then dX += dZ.Y^T and dY += X^T.dZ (beta = 1) from one call: "
                                 "the reference executor's literal fill + accumulate",
                     "ms_per_step": round(ems, 4), "ms_per_step_samples": [round(v, 4) for v in esamples],
                     "tflops": round(et, 2), "pct_mfma_peak": round(100.0 * et / PEAK[dtype], 2),
                     "frac": round(wl.flops / 3 / (eavg * 1e-3) / 1e12 / PEAK[dtype], 4), "launch_us": round(eavg * 1e3, 2)}

    form, note = "", None
    if is_mm or is_conv:
        form = ", fill + accumulate" if EAGER_ZERO else ", overwrite form"
        note = ("gradients: zero fill + accumulate (beta = 1), the reference executor's literal sequence" if EAGER_ZERO else
                "gradients: written by the overwrite form (beta = 0) that this build's executor issues while the zero fill "
                "of a gradient is still deferred -- same flops, same result as fill + accumulate"
                + (", which is reported beside it under eager_zero" if eager else ""))
    out = {
        "metric": "Conv2d fwd+bwd images/s" if is_conv else "%s fwd+bwd images/s" % wl.key if is_stream
        else "MatrixMultiply fwd+bwd TFLOP/s",
        "value": round(wl.B / (ms * 1e-3), 1) if is_conv or is_stream else round(tflops, 2),
        "unit": "images/s" if is_conv or is_stream else "TFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "settle_ms": SETTLE_MS, "ms_per_step": round(ms, 4),
        "reps": len(samples), "ms_per_step_samples": [round(v, 4) for v in samples],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "ALL-ZERO OPERANDS (diagnostic run, not a benchmark value)" if ZERO_OPERANDS else
        "synthetic (seeded numpy generators, resident in HBM before timing)",
        "config": {"workload": wl.name + form, **({"note": note} if note else {})},
        "pct_mfma_peak": None if is_stream else round(100.0 * tflops / PEAK[dtype], 2),
        "tflops": round(tflops, 2),
        "algorithmic_GBps": round(wl.bytes / (ms * 1e-3) / 1e9, 1),
        "parts": parts,
        "roofline": roof,
    }
    if eager:
        out["eager_zero"] = eager
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(a.workload)
    if not a.no_others:
        others = {}
        for key in ("c1", "c2a", "c2b", "c3", "f1", "f1s", "c4", "c4h", "c4e", "c4e_unfused", "c4x", "i4", "k5", "c5", "c5l", "e4", "p4", "d3"):
            if key == a.workload:
                continue
            del wl
            wl = make_workload(key)
            oms, _ = _time_steps(wl.step, 20, 3, reps=3)
            o = {"ms_per_step": round(oms, 4), "tflops": round(wl.flops / (oms * 1e-3) / 1e12, 2),
                 "algorithmic_GBps": round(wl.bytes / (oms * 1e-3) / 1e9, 1)}
            if isinstance(wl, (ConvWorkload, DeconvLiteralWorkload, BiasReluWorkload, PoolWorkload, GatherMapsWorkload, DeconvMapsWorkload)):
                o["images_per_s"] = round(wl.B / (oms * 1e-3), 1)
            if isinstance(wl, (GatherMapsWorkload, DeconvMapsWorkload)):  # the two kernels alone, against the HBM peak
                for pname, (fn, amount) in wl.parts().items():
                    pms = _time_events(fn, 100)
                    o[pname] = {"launch_us": round(pms * 1e3, 2), "algorithmic_GBps": round(amount / (pms * 1e-3) / 1e9, 1),
                                "frac_of_hbm_peak": round(amount / (pms * 1e-3) / 1e9 / HBM_PEAK, 4), **_traffic_fields(key, pname)}
            if key in ("c1", "c5") and not EAGER_ZERO:  # launch-latency bound steps: the same launches replayed from a HIP graph
                o["ms_per_step_graph_replay"] = round(graph_replay_ms(wl, 50, 5), 4)
            others[key] = o
        out["others"] = others
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
