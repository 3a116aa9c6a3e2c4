#!/usr/bin/env python3
"""Writes tests/golden/deep8_cpu_reference.npz: inputs and outputs of Deep8's own CPU (Eigen) path.

Run in the build container, where oracle/_ref/libdeep8_ref.so has been compiled from the reference
sources (`make -C oracle ref`):   python tests/golden/make_golden.py
Every array is float32.  Case names: mm<i>_*, conv<i>_*, deconv<i>_*, patch<i>_*, loss<i>_* (Minus,
L1Norm, L2Norm, ReduceMean, AXPBY), adam<i>_* (AdamUpdate), pool<i>_* (MaxPooling2d / AvgPooling2d); the geometry of case i is stored in <kind><i>_cfg.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402

MM = [((3, 12, 7), (1, 7, 9)), ((1, 11, 6), (4, 6)), ((3, 8, 5), (3, 5, 6)), ((1, 8, 5), (3, 5, 6)),
      ((3, 8, 5), (3, 5)), ((1, 16, 32), (1, 32, 24))]
# B, IH, IW, IC, OC, FH, FW, covered, sy, sx, dy, dx
CONV = [(2, 9, 9, 3, 4, 3, 3, 1, 1, 1, 1, 1), (1, 12, 12, 2, 3, 4, 4, 1, 2, 2, 2, 2), (2, 8, 7, 3, 2, 3, 3, 0, 1, 1, 1, 1),
        (1, 10, 10, 2, 2, 5, 5, 1, 1, 1, 1, 1), (1, 11, 11, 2, 3, 3, 3, 0, 2, 2, 2, 2)]
# B, IH, IW, IC, OC, FH, FW, covered, sy, sx
DECONV = [(2, 4, 4, 3, 2, 4, 4, 0, 3, 3), (2, 4, 4, 3, 2, 4, 4, 1, 3, 3), (1, 5, 5, 2, 3, 4, 4, 0, 2, 2),
          (1, 5, 5, 2, 3, 4, 4, 1, 2, 2), (1, 4, 5, 2, 2, 3, 3, 0, 1, 1)]
LOSS = [((3, 7), (3, 7), ()), ((2, 5, 6), (1, 6), (0,)), ((4, 3, 2, 5), (4, 1, 1, 5), (1, 3)), ((1, 33), (1, 1), (-1,)),
        ((2, 3, 4, 5, 6), (1, 3, 1, 5, 1), (0, 2, 4)), ((5, 64), (5, 64), (0,))]
POOL = [(2, 8, 8, 3, 2, 2, 0, 2, 2), (1, 9, 9, 4, 3, 3, 0, 2, 2), (2, 7, 7, 2, 3, 3, 1, 2, 2), (1, 6, 6, 5, 3, 3, 1, 1, 1),
        (1, 10, 10, 2, 4, 4, 1, 3, 3)]


def main():
    ref = oracle.ref
    if ref is None:
        raise SystemExit("oracle/_ref/libdeep8_ref.so is missing: run `make -C oracle ref` first")
    r = np.random.default_rng(20241125)
    out = {}
    u = lambda s: r.uniform(-1, 1, s).astype(np.float32)
    for i, (xs, ys) in enumerate(MM):
        x, y = u(xs), u(ys)
        z = ref.matmul(x, y)
        dz, dx0, dy0 = u(z.shape), u(xs), u(ys)
        out.update({"mm%d_x" % i: x, "mm%d_y" % i: y, "mm%d_z" % i: z, "mm%d_dz" % i: dz,
                    "mm%d_dx0" % i: dx0, "mm%d_dy0" % i: dy0,
                    "mm%d_dx" % i: ref.matmul_grad_x(x, y, dz, dx0), "mm%d_dy" % i: ref.matmul_grad_y(x, y, dz, dy0)})
    for i, c in enumerate(CONV):
        B, IH, IW, IC, OC, FH, FW, cov, sy, sx, dy, dx = c
        x, w = u((B, IH, IW, IC)), u((OC, FH, FW, IC))
        a = (bool(cov), sy, sx, dy, dx)
        z = ref.conv2d(x, w, *a)
        gz, gx0, gw0 = u(z.shape), u(x.shape), u(w.shape)
        OH, OW, pt, pl = oracle.port.conv2d_geometry(IH, IW, FH, FW, cov, sy, sx, dy, dx)
        rfh, rfw = FH + (FH - 1) * (dy - 1), FW + (FW - 1) * (dx - 1)
        py, px = max(0, (OH - 1) * sy + rfh - IH), max(0, (OW - 1) * sx + rfw - IW)
        # the patch matrix Conv2dCPUImpl contracts over (deep8/src/math/Conv2d.cpp:352-353)
        patches = ref.image_patches(x, FH, FW, sy, sx, dy, dx, 1, 1, py // 2, py - py // 2, px // 2, px - px // 2, OH, OW)
        out.update({"conv%d_cfg" % i: np.array(c, np.int32), "conv%d_x" % i: x, "conv%d_w" % i: w, "conv%d_z" % i: z,
                    "conv%d_gz" % i: gz, "conv%d_gx0" % i: gx0, "conv%d_gw0" % i: gw0,
                    "conv%d_gx" % i: ref.conv2d_grad_x(x, w, gz, *a, gx=gx0),
                    "conv%d_gw" % i: ref.conv2d_grad_y(x, w, gz, *a, gw=gw0), "conv%d_patches" % i: patches})
    for i, c in enumerate(DECONV):
        B, IH, IW, IC, OC, FH, FW, cov, sy, sx = c
        x, w = u((B, IH, IW, IC)), u((OC, FH, FW, IC))
        a = (bool(cov), sy, sx)
        z = ref.deconv2d(x, w, *a)
        gz, gx0, gw0 = u(z.shape), u(x.shape), u(w.shape)
        OH, OW, pt, pl = oracle.port.deconv2d_geometry(IH, IW, FH, FW, cov, sy, sx)
        # the patches DeConv2dGradXCPUImpl extracts from dz (deep8/src/math/DeConv2d.cpp:403-411)
        gpt, gpl = FH - 1 - pt, FW - 1 - pl
        gpb, gpr = (IH - 1) * sy + FH - OH - gpt, (IW - 1) * sx + FW - OW - gpl
        gpatches = ref.image_patches(gz, FH, FW, sy, sx, 1, 1, 1, 1, gpt, gpb, gpl, gpr, IH, IW)
        out.update({"deconv%d_cfg" % i: np.array(c, np.int32), "deconv%d_x" % i: x, "deconv%d_w" % i: w,
                    "deconv%d_z" % i: z, "deconv%d_gz" % i: gz, "deconv%d_gx0" % i: gx0, "deconv%d_gw0" % i: gw0,
                    "deconv%d_gx" % i: ref.deconv2d_grad_x(x, w, gz, *a, gx=gx0),
                    "deconv%d_gw" % i: ref.deconv2d_grad_y(x, w, gz, *a, gw=gw0), "deconv%d_gpatches" % i: gpatches})
    # Minus / L1Norm / L2Norm / ReduceMean / AXPBY: x shape, y shape (Minus operand), mean axes
    for i, (xs, ys, axes) in enumerate(LOSS):
        x, y = u(xs), u(ys)
        z = ref.minus(x, y)
        dz = u(z.shape)
        n1, n2 = ref.norm(1, x), ref.norm(2, x)
        dn, dx0, dy0 = u(n1.shape), u(xs), u(ys)
        m = ref.reduce_mean(x, axes)
        dm = u(m.shape)
        out.update({"loss%d_x" % i: x, "loss%d_y" % i: y, "loss%d_axes" % i: np.array(axes, np.int32), "loss%d_z" % i: z,
                    "loss%d_dz" % i: dz, "loss%d_dx0" % i: dx0, "loss%d_dy0" % i: dy0, "loss%d_dn" % i: dn, "loss%d_dm" % i: dm,
                    "loss%d_minus_gx" % i: ref.minus_grad(0, x, y, dz, dx0), "loss%d_minus_gy" % i: ref.minus_grad(1, x, y, dz, dy0),
                    "loss%d_l1" % i: n1, "loss%d_l2" % i: n2,
                    "loss%d_l1_gx" % i: ref.norm_grad(1, x, n1, dn, dx0), "loss%d_l2_gx" % i: ref.norm_grad(2, x, n2, dn, dx0),
                    "loss%d_mean" % i: m, "loss%d_mean_gx" % i: ref.reduce_mean_grad(x, m, dm, axes, dx=dx0),
                    "loss%d_axpby" % i: ref.axpby(x, -0.01, dx0, 0.999)})
    # AdamUpdate: three consecutive steps from the same state, with weight decay
    for i, n in enumerate((7, 64)):
        st = [u((1, n)), None, np.zeros((1, n), np.float32), np.zeros((1, n), np.float32)]
        out["adam%d_value0" % i] = st[0]
        for step in (1, 2, 3):
            g = u((1, n))
            out["adam%d_grad%d" % (i, step)] = g
            st = list(ref.adam_update(st[0], g, st[2], st[3], 0.9, 0.999, 1e-7, 0.01, 0.001, step))
            out["adam%d_step%d" % (i, step)] = np.stack(st)  # value, gradient (with the decay term), m, v
    # MaxPooling2d / AvgPooling2d: B, IH, IW, C, FH, FW, covered, sy, sx
    for i, c in enumerate(POOL):
        B, IH, IW, C, FH, FW, cov, sy, sx = c
        x = u((B, IH, IW, C))
        a = (FH, FW, bool(cov), sy, sx)
        ymax, yavg = ref.pool2d(True, x, *a), ref.pool2d(False, x, *a)
        dy, dx0 = u(ymax.shape), u(x.shape)
        out.update({"pool%d_cfg" % i: np.array(c, np.int32), "pool%d_x" % i: x, "pool%d_max" % i: ymax, "pool%d_avg" % i: yavg,
                    "pool%d_dy" % i: dy, "pool%d_dx0" % i: dx0,
                    "pool%d_max_gx" % i: ref.pool2d_grad(True, x, dy, *a, dx=dx0),
                    "pool%d_avg_gx" % i: ref.pool2d_grad(False, x, dy, *a, dx=dx0)})
    path = os.path.join(HERE, "deep8_cpu_reference.npz")
    np.savez_compressed(path, **out)
    print("wrote %s (%d arrays, %d bytes)" % (path, len(out), os.path.getsize(path)))


if __name__ == "__main__":
    main()
