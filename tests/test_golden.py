"""The committed fixtures (tests/golden/fixtures.npz, written by tests/golden/make_fixtures.py from the
reference tests' own generators): the oracle must still produce them (CPU), and the HIP path must produce
them through the C ABI (GPU)."""
import os
import sys

import numpy as np
import pytest

import oracle as orc

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_fixtures as mk  # noqa: E402  (the generators and the case selection, shared with the writer)

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.npz"))


def unpack(row, heads):
    row = [int(v) for v in row]
    return tuple(row[:heads]) + tuple((row[i], row[i + 1]) for i in range(heads, len(row), 2))


def test_oracle_reproduces_the_committed_fixtures():
    fresh = mk.build()
    assert sorted(fresh) == sorted(FIX.files)
    for k in FIX.files:
        assert fresh[k].dtype == FIX[k].dtype and np.array_equal(fresh[k], FIX[k]), k


def test_fixture_values_are_what_the_definitions_say():
    """Spot checks that do not go through the oracle: an im2col entry is the input element its index names, a
    pooled value is the window's maximum, a dot entry is the integer sum."""
    bs, c, ih, iw, f, p, s, d = unpack(FIX["im2col_cases"][1], 4)
    y = FIX["im2col_f32_1"]
    x = mk.ramp((bs, c, ih, iw))
    oh, ow = (ih + 2 * p[0] - d[0] * (f[0] - 1) - 1) // s[0] + 1, (iw + 2 * p[1] - d[1] * (f[1] - 1) - 1) // s[1] + 1
    assert y.shape == (bs * oh * ow, c * f[0] * f[1])
    for (b, ho, wo, ci, fi, fj) in [(0, 0, 0, 0, 0, 0), (bs - 1, oh - 1, ow - 1, c - 1, f[0] - 1, f[1] - 1)]:
        hi, wi = -p[0] + fi * d[0] + s[0] * ho, -p[1] + fj * d[1] + s[1] * wo
        want = x[b, ci, hi, wi] if 0 <= hi < ih and 0 <= wi < iw else 0.0
        assert y[(b * oh + ho) * ow + wo, (ci * f[0] + fi) * f[1] + fj] == want
    x = mk.cyc((1, 1, 4, 4), 10)
    assert np.array_equal(FIX["pool_f32_0"][0, 0], x[0, 0].reshape(2, 2, 2, 2).transpose(0, 2, 1, 3).reshape(2, 2, 4).max(-1))
    a = mk.cyc((4, 4), 9, 1).astype(np.int64)
    assert np.array_equal(FIX["dot_f32_4_01"].astype(np.int64), a @ a.T)


@pytest.mark.gpu
def test_hip_path_reproduces_the_committed_fixtures():
    import autograph_amd as ag
    ag.Device(0)
    for dtype in ("f32", "bf16"):
        for n, row in enumerate(FIX["im2col_cases"]):
            bs, c, ih, iw, f, p, s, d = unpack(row, 4)
            x = mk.to_dtype(mk.ramp((bs, c, ih, iw)), dtype)
            opts = ag.Im2ColConv2Options(filter=f, padding=p, stride=s, dilation=d)
            y = ag.Tensor.from_array(x).im2col_conv2(opts).into_array()
            assert np.array_equal(y, FIX[f"im2col_{dtype}_{n}"]), ("im2col", dtype, n)
            oh, ow = opts.output_shape((ih, iw))
            g = mk.to_dtype(mk.ramp(y.shape), dtype)
            dx = ag.Tensor.from_array(g).col2im_conv2(ag.Col2ImConv2Options((oh, ow), f, p, s, d)).into_array()
            assert np.array_equal(dx, FIX[f"col2im_{dtype}_{n}"]), ("col2im", dtype, n)
        popts = ag.MaxPool2Options((2, 2), (2, 2))
        for n, shape in enumerate(mk.POOL_SHAPES):
            x = mk.to_dtype(mk.cyc(shape, 10), dtype)
            tx = ag.Tensor.from_array(x)
            y = tx.max_pool2(popts).into_array()
            assert np.array_equal(y, FIX[f"pool_{dtype}_{n}"]), ("pool", dtype, n)
            dy = mk.to_dtype(np.arange(y.size, dtype=np.float32).reshape(y.shape), dtype)
            dxt = tx.clone()
            dxt.max_pool2_backward(ag.Tensor.from_array(dy), popts)
            assert np.array_equal(dxt.into_array(), FIX[f"pool_bwd_{dtype}_{n}"]), ("pool_bwd", dtype, n)
        for n in (2, 4, 5, 8, 16):
            a = mk.to_dtype(mk.cyc((n, n), 9, 1), dtype)
            t = ag.Tensor.from_array(a)
            for ta in (0, 1):
                for tb in (0, 1):
                    got = (t.t() if ta else t).dot(t.t() if tb else t).into_array()
                    assert np.array_equal(got, FIX[f"dot_{dtype}_{n}_{ta}{tb}"]), ("dot", dtype, n, ta, tb)
    for n, row in enumerate(FIX["conv_cases"]):
        bs, ic, oc, ih, iw, f, p, s, d = unpack(row, 5)
        x, w = mk.cyc((bs, ic, ih, iw), 10, 1), mk.cyc((oc, ic) + tuple(f), 10, 1)
        for fn in (ag.conv2_im2col_forward, ag.conv2_direct_forward):
            y = fn(ag.Tensor.from_array(x), ag.Tensor.from_array(w), padding=p, stride=s, dilation=d).into_array()
            assert np.array_equal(y, FIX[f"conv_{n}"]), ("conv", n, fn.__name__)
