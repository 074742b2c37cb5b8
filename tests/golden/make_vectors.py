#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: seeded inputs and expected outputs of the delta operators.

The reference holds no golden vectors for this path and cannot be built here, so the
expected outputs come from the loop-level numpy statements in bruteforce.py (nothing from
`oracle/` and nothing from the HIP library is involved).  Inputs are fp32 and, for the
elementwise operators, also fp16 (their results are defined bit for bit; contractions carry an
expectation accumulated in float64 (stored as fp32) that fp32 / fp16 results are compared with under the stated tolerance).

    python tests/golden/make_vectors.py        # rewrites vectors.npz next to this file
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import bruteforce as bf  # noqa: E402

CONVS = {
    # name: (cin, cout, kernel, stride, padding, dilation, groups, H, W)
    "conv3x3": (8, 12, (3, 3), (1, 1), (1, 1), (1, 1), 1, 10, 9),
    "conv3x3s2": (8, 8, (3, 3), (2, 2), (1, 1), (1, 1), 1, 11, 10),
    "conv1x1": (16, 24, (1, 1), (1, 1), (0, 0), (1, 1), 1, 9, 9),
    "dw3x3": (16, 16, (3, 3), (1, 1), (1, 1), (1, 1), 16, 9, 10),
    "dw3x3s2": (16, 16, (3, 3), (2, 2), (1, 1), (1, 1), 16, 10, 10),
    "conv3x3d2": (4, 6, (3, 3), (1, 1), (2, 2), (2, 2), 1, 9, 9),
    "stem": (3, 8, (3, 3), (2, 2), (1, 1), (1, 1), 1, 12, 12),
}
DECONVS = {"deconv4s2": (8, 6, 4, 2, 1, 6, 7), "deconv6s4": (4, 4, 6, 4, 1, 4, 5)}
POOLS = {"max2s2": ((2, 2), (2, 2), (0, 0), 0), "max3s2p1": ((3, 3), (2, 2), (1, 1), 0),
         "avg2s2": ((2, 2), (2, 2), (0, 0), 1), "avg_global": ((6, 6), (1, 1), (0, 0), 1),
         "max3s2_asym": ((3, 3), (2, 2), (0, 1, 0, 1), 0)}


def half_exact(a):
    """Values representable in fp16 so that fp32 and fp16 runs start from identical inputs."""
    return a.astype(np.float16).astype(np.float32)


def main():
    rng = np.random.default_rng(20240)
    out = {}
    for name, (ci, co, k, s, p, d, g, H, W) in CONVS.items():
        x = half_exact(rng.standard_normal((2, ci, H, W)))
        m = (rng.random((2, 1, H, W)) < 0.3).astype(np.int32)
        w = half_exact(rng.standard_normal((co, ci // g, *k)) / np.sqrt(ci // g * k[0] * k[1]))
        b = half_exact(rng.standard_normal(co))
        y, om = bf.conv(x, m, w, b, s, p, d, g)
        out.update({f"{name}.x": x, f"{name}.mask": m, f"{name}.w": w, f"{name}.b": b,
                    f"{name}.out": y.astype(np.float32), f"{name}.out_mask": om,
                    f"{name}.cfg": np.array([*s, *bf.pad4(p), *d, g], np.int64)})
    for name, (ci, co, k, s, p, H, W) in DECONVS.items():
        x = half_exact(rng.standard_normal((2, ci, H, W)))
        m = (rng.random((2, 1, H, W)) < 0.3).astype(np.int32)
        w = half_exact(rng.standard_normal((ci, co, k, k)) / np.sqrt(ci * k * k))
        b = half_exact(rng.standard_normal(co))
        y, om = bf.deconv(x, m, w, b, (s, s), (p, p))
        out.update({f"{name}.x": x, f"{name}.mask": m, f"{name}.w": w, f"{name}.b": b,
                    f"{name}.out": y.astype(np.float32), f"{name}.out_mask": om,
                    f"{name}.cfg": np.array([s, p], np.int64)})
    for name, (k, s, p, mode) in POOLS.items():
        x = half_exact(rng.standard_normal((2, 8, 6, 6)))
        prev = half_exact(rng.standard_normal((2, 8, 6, 6)))
        m = (rng.random((2, 1, 6, 6)) < 0.3).astype(np.int32)
        y, om = bf.pool(x, prev, m, k, s, p, mode)
        out.update({f"{name}.x": x, f"{name}.prev": prev, f"{name}.mask": m,
                    f"{name}.out": y.astype(np.float32), f"{name}.out_mask": om,
                    f"{name}.cfg": np.array([*k, *s, *bf.pad4(p), mode], np.int64)})
    for dt, tag in ((np.float32, "f32"), (np.float16, "f16")):
        for C in (3, 8, 33):
            x = rng.standard_normal((2, C, 7, 6)).astype(dt)
            noise = rng.standard_normal(x.shape) * (rng.random((2, 1, 7, 6)) < 0.4) * 0.3
            prev = (x + noise).astype(dt)
            dd = np.abs((x - prev).astype(dt))
            prev = np.where((dd > 0.09) & (dd < 0.11), x, prev).astype(dt)  # no near-ties (fp16 even-C rule)
            delta, mask, new_prev = bf.sparsify(x, prev, 0.1)
            n = f"sparsify_{tag}_c{C}"
            out.update({f"{n}.x": x, f"{n}.prev": prev, f"{n}.delta": delta, f"{n}.mask": mask,
                        f"{n}.new_prev": new_prev})
            for act in (1, 2, 3):
                scale = (rng.random((2, 1, 7, 6)) < 0.5) * 0.97 + 0.03
                delta = (rng.standard_normal(x.shape) * scale).astype(dt)
                prev = (rng.standard_normal(x.shape) * 3).astype(dt)
                trunc = (rng.standard_normal(x.shape) * 0.02).astype(dt)
                mask = (rng.random((2, 1, 7, 6)) < 0.7).astype(np.int32)
                r = bf.activate_truncate(delta, prev, trunc, mask, 0.05, act)
                n = f"act{act}_{tag}_c{C}"
                out.update({f"{n}.delta": delta, f"{n}.prev": prev, f"{n}.trunc": trunc, f"{n}.mask": mask,
                            f"{n}.out_delta": r[0], f"{n}.out_prev": r[1], f"{n}.out_trunc": r[2],
                            f"{n}.out_mask": r[3]})
            a = rng.standard_normal(x.shape).astype(dt)
            b = rng.standard_normal(x.shape).astype(dt)
            ma = (rng.random((2, 1, 7, 6)) < 0.5).astype(np.int32)
            mb = (rng.random((2, 1, 7, 6)) < 0.5).astype(np.int32)
            y, mo = bf.add(a, ma, b, mb, 0.75, 1.5)
            n = f"add_{tag}_c{C}"
            out.update({f"{n}.a": a, f"{n}.b": b, f"{n}.mask_a": ma, f"{n}.mask_b": mb, f"{n}.out": y,
                        f"{n}.out_mask": mo})
    np.savez_compressed(os.path.join(HERE, "vectors.npz"), **out)
    print(f"{len(out)} arrays -> vectors.npz")


if __name__ == "__main__":
    main()
