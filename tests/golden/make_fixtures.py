#!/usr/bin/env python3
"""Writes tests/golden/fixtures.npz: expected outputs, computed by the CPU oracle, for inputs built with the
generators the reference's own tests use (integer ramps and cycles, tests/integration_tests.rs:291-305, :885-923,
:1041-1046, :1499-1628).  The reference holds no binary vectors for this path, only those generators, so the
fixtures pin (1) the oracle against later edits and (2) the HIP path against data that travels with the tests.

    python3 tests/golden/make_fixtures.py

Inputs are not stored (the tests rebuild them from the case parameters kept in the file); only small cases are
taken: every 101st case of the im2col / col2im grid, the four pooling shapes, dot sizes up to 16, every 27th conv2 case.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))            # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))  # repo root

import oracle as orc  # noqa: E402
from refgrid import BATCH_IN_OUT, POOL_SHAPES, cases, conv_options, input_shapes  # noqa: E402


def ramp(shape):      # 1..=len (integration_tests.rs:1499-1512)
    return np.arange(1, int(np.prod(shape)) + 1, dtype=np.float32).reshape(shape)


def cyc(shape, m, base=0):   # (base..base+m).cycle()
    return ((np.arange(int(np.prod(shape))) % m) + base).astype(np.float32).reshape(shape)


def to_dtype(x, dtype):
    return orc.f32_to_bf16(x) if dtype == "bf16" else np.ascontiguousarray(x, dtype=np.float32)


def build():
    out = {}
    im2col_cases = [c for i, c in enumerate(cases()) if i % 101 == 0]
    out["im2col_cases"] = np.array([[bs, c, ih, iw, *f, *p, *s, *d] for bs, c, ih, iw, f, p, s, d in im2col_cases], dtype=np.int32)
    for dtype in ("f32", "bf16"):
        for n, (bs, c, ih, iw, f, p, s, d) in enumerate(im2col_cases):
            x = to_dtype(ramp((bs, c, ih, iw)), dtype)
            y = orc.im2col_conv2(x, f, p, s, d)
            out[f"im2col_{dtype}_{n}"] = y
            oh, ow = orc.conv_out(ih, f[0], p[0], s[0], d[0]), orc.conv_out(iw, f[1], p[1], s[1], d[1])
            g = to_dtype(ramp(y.shape), dtype)
            out[f"col2im_{dtype}_{n}"] = orc.col2im_conv2(g, (oh, ow), f, p, s, d)
        for n, shape in enumerate(POOL_SHAPES):
            x = to_dtype(cyc(shape, 10), dtype)
            y = orc.max_pool2(x, (2, 2))
            out[f"pool_{dtype}_{n}"] = y
            dy = to_dtype(np.arange(y.size, dtype=np.float32).reshape(y.shape), dtype)
            out[f"pool_bwd_{dtype}_{n}"] = orc.max_pool2_backward(x, dy, (2, 2))
        for n in (2, 4, 5, 8, 16):
            a = to_dtype(cyc((n, n), 9, 1), dtype)
            for ta in (0, 1):
                for tb in (0, 1):
                    av, bv = (a.T if ta else a), (a.T if tb else a)
                    want = orc.gemm_bf16_f32acc(av, bv) if dtype == "bf16" else orc.gemm_f64acc(av, bv).astype(np.float32)
                    out[f"dot_{dtype}_{n}_{ta}{tb}"] = want
    conv_cases = []
    for f, p, s, d in conv_options():
        for ih, iw in list(input_shapes(f, p, s, d))[::3]:
            for bs, ic, oc in BATCH_IN_OUT:
                conv_cases.append((bs, ic, oc, ih, iw, f, p, s, d))
    conv_cases = conv_cases[::27]
    out["conv_cases"] = np.array([[bs, ic, oc, ih, iw, *f, *p, *s, *d] for bs, ic, oc, ih, iw, f, p, s, d in conv_cases], dtype=np.int32)
    for n, (bs, ic, oc, ih, iw, f, p, s, d) in enumerate(conv_cases):
        x, w = cyc((bs, ic, ih, iw), 10, 1), cyc((oc, ic) + tuple(f), 10, 1)
        out[f"conv_{n}"] = orc.conv2_naive_f64(x, w, p, s, d).astype(np.float32)  # exact integers below 2^24
    return out


if __name__ == "__main__":
    data = build()
    path = os.path.join(HERE, "fixtures.npz")
    np.savez_compressed(path, **data)
    print(f"{path}: {len(data)} arrays, {os.path.getsize(path) / 1024:.1f} KiB")
