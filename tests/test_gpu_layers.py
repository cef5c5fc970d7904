"""Layer-level parity on the GPU: Conv2 (im2col chain and direct kernel), fused ReLU/MaxPool2,
Dense, and the LeNet5 forward pass of the reference's benchmark, against the CPU oracle.

Mirrors conv2_im2col_<T>_<opts> (tests/integration_tests.rs:986-993, body :1182-1251), which
checks the chain against the naive 7-deep loop on x, w = (1..=10).cycle() data.
"""
import ctypes as C

import numpy as np
import pytest

import oracle as orc
from refgrid import BATCH_IN_OUT, conv_options, input_shapes

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ag():
    import autograph_amd as ag
    ag.Device(0)
    return ag


def to_dtype(x, dtype):
    return orc.f32_to_bf16(x) if dtype == "bf16" else np.ascontiguousarray(x, dtype=np.float32)


def as_f32(x):
    return orc.bf16_to_f32(x) if x.dtype == np.uint16 else x


def cyc10(shape):
    return ((np.arange(int(np.prod(shape))) % 10) + 1).astype(np.float32).reshape(shape)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("alg", ["im2col", "direct"])
def test_conv2_reference_grid(ag, dtype, alg):
    """Whole filter/padding/stride/dilation grid x (batch, inputs, outputs) list; exact-integer data.
    f32 must be exact (all sums < 2^24); bf16 must be the correctly rounded exact sum."""
    n = 0
    for f, p, s, d in conv_options():
        for ih, iw in list(input_shapes(f, p, s, d))[::3]:
            for bs, ic, oc in BATCH_IN_OUT:
                x = to_dtype(cyc10((bs, ic, ih, iw)), dtype)
                w = to_dtype(cyc10((oc, ic) + f), dtype)
                want = orc.conv2_naive_f64(as_f32(x), as_f32(w), p, s, d)
                fn = ag.conv2_im2col_forward if alg == "im2col" else ag.conv2_direct_forward
                y = fn(ag.Tensor.from_array(x), ag.Tensor.from_array(w), padding=p, stride=s, dilation=d).into_array()
                assert y.shape == want.shape
                if dtype == "f32":
                    assert np.array_equal(y.astype(np.float64), want), (alg, bs, ic, oc, ih, iw, f, p, s, d)
                else:
                    # f32 accumulation of these integers is exact, so the result is the single RNE
                    # rounding of the exact sum (the reference compares two bf16 computations with
                    # epsilon = fh*fw, :1239-1243; this is the tighter statement)
                    assert np.array_equal(y, orc.f32_to_bf16(want.astype(np.float32))), (alg, bs, ic, oc, ih, iw, f, p, s, d)
                n += 1
    assert n > 500


CONV_SEEDED = [
    # bs, ic, ih, iw, oc, filter, padding, stride, dilation
    (100, 1, 28, 28, 6, (5, 5), (0, 0), (1, 1), (1, 1)),    # LeNet5 conv1
    (100, 6, 12, 12, 16, (5, 5), (0, 0), (1, 1), (1, 1)),   # LeNet5 conv2
    (8, 16, 20, 20, 32, (3, 3), (1, 1), (1, 1), (1, 1)),
    (3, 5, 17, 23, 7, (3, 5), (2, 1), (2, 3), (2, 1)),
    (4, 64, 14, 14, 128, (3, 3), (1, 1), (1, 1), (1, 1)),   # config-3 shaped, small batch
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", CONV_SEEDED)
def test_conv2_seeded_both_algorithms(ag, dtype, case):
    bs, ic, ih, iw, oc, f, p, s, d = case
    rng = np.random.default_rng(21)
    x = to_dtype(rng.standard_normal((bs, ic, ih, iw)), dtype)
    w = to_dtype(rng.standard_normal((oc, ic) + f) * np.sqrt(2.0 / (ic * f[0] * f[1])), dtype)
    b = to_dtype(rng.standard_normal(oc) * 0.1, dtype)
    want = orc.conv2_naive_f64(as_f32(x), as_f32(w), p, s, d)
    scale = orc.conv2_naive_f64(np.abs(as_f32(x)), np.abs(as_f32(w)), p, s, d)
    k = ic * f[0] * f[1]
    tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
    for alg in ("im2col", "direct"):
        fn = ag.conv2_im2col_forward if alg == "im2col" else ag.conv2_direct_forward
        try:
            y = fn(tx, tw, padding=p, stride=s, dilation=d).into_array()
        except ag.AghError as e:
            assert alg == "direct" and e.code == -4  # does not fit in LDS: documented fallback
            continue
        got = as_f32(y).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * scale + 1e-30), alg
        else:
            ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0**-126))) - 7)
            assert np.all(np.abs(got - want) <= ulp + 1e-2 * np.abs(want) + 8 * np.sqrt(k) * 2.0**-24 * scale), alg
        # bias + relu epilogue: equals the separate ops applied to this very conv result, bit for bit
        yb = fn(tx, tw, padding=p, stride=s, dilation=d, bias=tb, relu=True).into_array()
        n, c, h, wd = y.shape
        flat = np.ascontiguousarray(y.transpose(0, 2, 3, 1).reshape(-1, c))
        ref = orc.relu(orc.bias_add_rows(flat, b)).reshape(n, h, wd, c).transpose(0, 3, 1, 2)
        assert np.array_equal(yb, ref), alg


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_conv2_direct_fused_relu_pool(ag, dtype):
    """conv -> Relu -> MaxPool2(2x2) in one launch equals the three layers applied to the conv result."""
    rng = np.random.default_rng(22)
    for (bs, ic, ih, iw, oc, f) in [(100, 1, 28, 28, 6, (5, 5)), (100, 6, 12, 12, 16, (5, 5)), (5, 3, 11, 9, 10, (3, 3))]:
        x = to_dtype(rng.uniform(0, 1, (bs, ic, ih, iw)), dtype)
        w = to_dtype(rng.uniform(-1, 1, (oc, ic) + f) * np.sqrt(2.0 / (ic * f[0] * f[1])), dtype)
        tx, tw = ag.Tensor.from_array(x), ag.Tensor.from_array(w)
        conv = ag.conv2_direct_forward(tx, tw).into_array()
        fused = ag.conv2_direct_forward(tx, tw, relu=True, pool2x2=True).into_array()
        assert np.array_equal(fused, orc.max_pool2(orc.relu(conv), (2, 2)))


CONV_MFMA = [
    # bs, ic, ih, iw, oc, filter, padding: shapes the implicit-GEMM (matrix core) convolution takes
    (2, 64, 56, 56, 128, (3, 3), (1, 1)),    # config-3 layer, small batch
    (3, 16, 24, 24, 64, (5, 5), (0, 0)),     # one 16-channel step per tap, partial last tile (400 positions)
    (2, 32, 16, 16, 192, (3, 3), (1, 1)),    # two output-channel tiles, the second half empty
    (1, 128, 8, 32, 64, (1, 1), (0, 0)),     # 1x1, staged tile exactly 64 KB
    (2, 16, 20, 16, 64, (3, 5), (1, 2)),     # rectangular filter, unequal padding, odd step count (15)
    (1, 128, 56, 56, 64, (3, 3), (1, 1)),    # rows of 128 channels exceed half a CU's LDS: two passes of 64 channels
    (2, 96, 16, 24, 64, (3, 3), (1, 1)),     # channel count not a power of two: three passes of 32
]


@pytest.mark.parametrize("case", CONV_MFMA)
def test_conv2_direct_bf16_matrix_core_path(ag, case):
    bs, ic, ih, iw, oc, f, p = case
    rng = np.random.default_rng(25)
    x = orc.f32_to_bf16(rng.standard_normal((bs, ic, ih, iw)).astype(np.float32))
    w = orc.f32_to_bf16((rng.standard_normal((oc, ic) + f) * np.sqrt(2.0 / (ic * f[0] * f[1]))).astype(np.float32))
    b = orc.f32_to_bf16((rng.standard_normal(oc) * 0.1).astype(np.float32))
    tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
    y = ag.conv2_direct_forward(tx, tw, padding=p).into_array()
    want = orc.conv2_naive_f64(orc.bf16_to_f32(x), orc.bf16_to_f32(w), p, (1, 1), (1, 1))
    scale = orc.conv2_naive_f64(np.abs(orc.bf16_to_f32(x)), np.abs(orc.bf16_to_f32(w)), p, (1, 1), (1, 1))
    assert y.shape == want.shape
    k = ic * f[0] * f[1]
    got = orc.bf16_to_f32(y).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0**-126))) - 7)
    assert np.all(np.abs(got - want) <= ulp + 1e-2 * np.abs(want) + 8 * np.sqrt(k) * 2.0**-24 * scale)
    # and against the im2col + GEMM chain: same f32 sums in another order, so at most one bf16 step apart
    chain = orc.bf16_to_f32(ag.conv2_im2col_forward(tx, tw, padding=p).into_array()).astype(np.float64)
    assert np.all(np.abs(got - chain) <= 2 * ulp + 16 * np.sqrt(k) * 2.0**-24 * scale)
    assert np.mean(got != chain) < 0.2
    # bias + relu epilogue: equals the separate ops applied to this very conv result, bit for bit
    yb = ag.conv2_direct_forward(tx, tw, padding=p, bias=tb, relu=True).into_array()
    n, c, h, wd = y.shape
    flat = np.ascontiguousarray(y.transpose(0, 2, 3, 1).reshape(-1, c))
    ref = orc.relu(orc.bias_add_rows(flat, b)).reshape(n, h, wd, c).transpose(0, 3, 1, 2)
    assert np.array_equal(yb, ref)
    # exact-integer data: every sum is exact in f32, so the result is the single RNE rounding of it
    xi = orc.f32_to_bf16(((np.arange(x.size) % 10) + 1).astype(np.float32).reshape(x.shape))
    wi = orc.f32_to_bf16(((np.arange(w.size) % 7) - 3).astype(np.float32).reshape(w.shape))
    yi = ag.conv2_direct_forward(ag.Tensor.from_array(xi), ag.Tensor.from_array(wi), padding=p).into_array()
    exact = orc.conv2_naive_f64(orc.bf16_to_f32(xi), orc.bf16_to_f32(wi), p, (1, 1), (1, 1))
    assert np.array_equal(yi, orc.f32_to_bf16(exact.astype(np.float32)))


CONV_FEW_CHANNELS = [
    # bs, ic, ih, iw, oc, filter, padding: layers the 16-channel-wide matrix-core kernel takes (or can be made to)
    (100, 6, 12, 12, 16, (5, 5), (0, 0)),    # LeNet5 conv2: 150 taps (5 chunks, 10 padded), 4 tiles of 4 windows
    (100, 1, 28, 28, 6, (5, 5), (0, 0)),     # LeNet5 conv1: 6 of 16 columns live, 25 taps in one chunk, 36 tiles
    (7, 3, 11, 9, 10, (3, 3), (1, 1)),       # padding, odd sizes: last tile partly empty, pooling drops a row and a column
    (5, 8, 9, 14, 16, (3, 5), (2, 1)),       # rectangular filter, padding larger than half the filter
    (3, 20, 6, 6, 12, (1, 1), (0, 0)),       # 1x1: the tap table is the channel stride
    (2, 4, 40, 36, 9, (3, 3), (0, 0)),       # many tiles per image: 4 tiles per unit
    (300, 2, 5, 5, 3, (2, 2), (0, 0)),       # tiny images, many per workgroup
]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("case", CONV_FEW_CHANNELS)
def test_conv2_direct_few_channels_matrix_core_path(ag, monkeypatch, dtype, case):
    """AGH_CONV_SMALL=1 sends every layer with at most 16 output channels through the 16x16x4 MFMA kernel (by itself
    the library picks it from 8 output channels and 32 taps).  Checked against the f64 convolution, exactly on integer
    data, and its fused bias / ReLU / 2x2 pool against the separate layers applied to its own plain result."""
    bs, ic, ih, iw, oc, f, p = case
    monkeypatch.setenv("AGH_CONV_SMALL", "1")
    rng = np.random.default_rng(27)
    x = to_dtype(rng.standard_normal((bs, ic, ih, iw)), dtype)
    w = to_dtype(rng.standard_normal((oc, ic) + f) * np.sqrt(2.0 / (ic * f[0] * f[1])), dtype)
    b = to_dtype(rng.standard_normal(oc) * 0.1, dtype)
    tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
    y = ag.conv2_direct_forward(tx, tw, padding=p).into_array()
    want = orc.conv2_naive_f64(as_f32(x), as_f32(w), p, (1, 1), (1, 1))
    scale = orc.conv2_naive_f64(np.abs(as_f32(x)), np.abs(as_f32(w)), p, (1, 1), (1, 1))
    assert y.shape == want.shape
    k = ic * f[0] * f[1]
    got = as_f32(y).astype(np.float64)
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0**-126))) - (7 if dtype == "bf16" else 23))
    assert np.all(np.abs(got - want) <= ulp + 8 * np.sqrt(k) * 2.0**-24 * scale)
    # the other kernel (register tiles on the vector units) sums the same products in another order
    monkeypatch.setenv("AGH_CONV_SMALL", "0")
    other = as_f32(ag.conv2_direct_forward(tx, tw, padding=p).into_array()).astype(np.float64)
    monkeypatch.setenv("AGH_CONV_SMALL", "1")
    assert np.all(np.abs(got - other) <= 2 * ulp + 16 * np.sqrt(k) * 2.0**-24 * scale)
    # epilogues, bit for bit on this kernel's own sums
    yb = ag.conv2_direct_forward(tx, tw, padding=p, bias=tb, relu=True).into_array()
    n, c, h, wd = y.shape
    flat = np.ascontiguousarray(y.transpose(0, 2, 3, 1).reshape(-1, c))
    ref = orc.relu(orc.bias_add_rows(flat, b)).reshape(n, h, wd, c).transpose(0, 3, 1, 2)
    assert np.array_equal(yb, ref)
    if h >= 2 and wd >= 2:
        fused = ag.conv2_direct_forward(tx, tw, padding=p, relu=True, pool2x2=True).into_array()
        assert np.array_equal(fused, orc.max_pool2(orc.relu(y), (2, 2)))
        fused_b = ag.conv2_direct_forward(tx, tw, padding=p, bias=tb, relu=True, pool2x2=True).into_array()
        assert np.array_equal(fused_b, orc.max_pool2(ref, (2, 2)))
    # exact-integer data: every sum is exact in f32
    xi = to_dtype(((np.arange(x.size) % 10) + 1).astype(np.float32).reshape(x.shape), dtype)
    wi = to_dtype(((np.arange(w.size) % 7) - 3).astype(np.float32).reshape(w.shape), dtype)
    yi = ag.conv2_direct_forward(ag.Tensor.from_array(xi), ag.Tensor.from_array(wi), padding=p).into_array()
    exact = orc.conv2_naive_f64(as_f32(xi), as_f32(wi), p, (1, 1), (1, 1)).astype(np.float32)
    assert np.array_equal(yi, to_dtype(exact, dtype))
    # an infinite input value reaches exactly the outputs whose window covers it: the padded taps behind the last one
    # (zeros of the filter bank) must not turn it into NaN anywhere
    xinf = np.abs(as_f32(x)).copy()
    xinf[0, ic - 1, ih // 2, iw // 2] = np.inf
    wpos = np.abs(as_f32(w)) + 0.01
    yinf = as_f32(ag.conv2_direct_forward(ag.Tensor.from_array(to_dtype(xinf, dtype)), ag.Tensor.from_array(to_dtype(wpos, dtype)),
                                          padding=p).into_array())
    want_inf = np.isinf(orc.conv2_naive_f64(as_f32(to_dtype(xinf, dtype)), as_f32(to_dtype(wpos, dtype)), p, (1, 1), (1, 1)))
    assert not np.isnan(yinf).any()
    assert np.array_equal(np.isinf(yinf), want_inf) and want_inf.any()


CONV_MFMA_F32 = [
    # the f32 variant steps 8 channels at a time
    (2, 64, 56, 56, 128, (3, 3), (1, 1)),    # config-3 layer, small batch: two passes of 32 channels
    (3, 8, 24, 24, 64, (5, 5), (0, 0)),      # one 8-channel step per tap, partial last tile (400 positions)
    (2, 32, 16, 16, 192, (3, 3), (1, 1)),    # two output-channel tiles, the second half empty
    (1, 128, 8, 32, 64, (1, 1), (0, 0)),     # 1x1
    (2, 16, 20, 16, 64, (3, 5), (1, 2)),     # rectangular filter, unequal padding, odd step count (30 = 4*7 + 2)
    (1, 16, 12, 28, 64, (3, 3), (0, 0)),     # width a multiple of 4 only, 260 positions (a 4-position tail tile)
    (1, 24, 20, 20, 64, (3, 3), (1, 1)),     # three passes of 8 channels
    (1, 256, 28, 28, 64, (3, 3), (1, 1)),    # four passes of 64 channels
]


@pytest.mark.parametrize("case", CONV_MFMA_F32)
def test_conv2_direct_f32_matrix_core_path(ag, case):
    bs, ic, ih, iw, oc, f, p = case
    rng = np.random.default_rng(26)
    x = rng.standard_normal((bs, ic, ih, iw)).astype(np.float32)
    w = (rng.standard_normal((oc, ic) + f) * np.sqrt(2.0 / (ic * f[0] * f[1]))).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
    y = ag.conv2_direct_forward(tx, tw, padding=p).into_array()
    want = orc.conv2_naive_f64(x, w, p, (1, 1), (1, 1))
    scale = orc.conv2_naive_f64(np.abs(x), np.abs(w), p, (1, 1), (1, 1))
    assert y.shape == want.shape
    k = ic * f[0] * f[1]
    # f32 products and sums: the GEMM bound, 1e-5 * sqrt(K) relative to the sum of magnitudes
    assert np.all(np.abs(y.astype(np.float64) - want) <= 1e-5 * np.sqrt(k) * np.maximum(scale, 1e-30))
    chain = ag.conv2_im2col_forward(tx, tw, padding=p).into_array()
    assert np.all(np.abs(y.astype(np.float64) - chain) <= 2e-5 * np.sqrt(k) * np.maximum(scale, 1e-30))
    # bias + relu epilogue: equals the separate ops applied to this very conv result, bit for bit
    yb = ag.conv2_direct_forward(tx, tw, padding=p, bias=tb, relu=True).into_array()
    n, c, h, wd = y.shape
    flat = np.ascontiguousarray(y.transpose(0, 2, 3, 1).reshape(-1, c))
    ref = orc.relu(orc.bias_add_rows(flat, b)).reshape(n, h, wd, c).transpose(0, 3, 1, 2)
    assert np.array_equal(yb, ref)
    # exact-integer data: every product and partial sum is an integer below 2^24, so any order gives the exact result
    xi = ((np.arange(x.size) % 10) + 1).astype(np.float32).reshape(x.shape)
    wi = ((np.arange(w.size) % 7) - 3).astype(np.float32).reshape(w.shape)
    yi = ag.conv2_direct_forward(ag.Tensor.from_array(xi), ag.Tensor.from_array(wi), padding=p).into_array()
    assert np.array_equal(yi, orc.conv2_naive_f64(xi, wi, p, (1, 1), (1, 1)).astype(np.float32))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_conv2_forward_config3_full_size(ag, dtype):
    """Conv2 forward of the benchmark list at full size (layer.rs:950-1005): batch 256, 64 -> 128 channels, 56x56,
    3x3, stride 1, pad 1, both algorithms (im2col + the 802816 x 576 x 128 GEMM, and the implicit GEMM with its
    3328 tiles walked XCD by XCD).  The oracle's naive f64 convolution is run on the 3x3 windows of sampled
    output positions (all 128 channels each): the four borders and corners of images, the first and last
    position of every tile of images that begin or end an XCD's run of tiles, and random ones.  The fused
    bias + ReLU launch equals the separate ops on the same result bit for bit."""
    bs, ic, ih, iw, oc = 256, 64, 56, 56, 128
    rng = np.random.default_rng(29)
    x = to_dtype(rng.standard_normal((bs, ic, ih, iw), dtype=np.float32), dtype)
    w = to_dtype((rng.standard_normal((oc, ic, 3, 3)) * np.sqrt(2.0 / (ic * 9))).astype(np.float32), dtype)
    b = to_dtype((rng.standard_normal(oc) * 0.1).astype(np.float32), dtype)
    xf, wf = as_f32(x), as_f32(w)
    # sampled (image, row, column)
    pts = []
    edge_imgs = [0, 1, 31, 32, 63, 64, 127, 128, 191, 192, 223, 224, 254, 255]
    for img in edge_imgs:
        for pos in sorted({0, 55, 56, 3080, 3135} | {t * 256 for t in range(13)} | {t * 256 - 1 for t in range(1, 13)}):
            pts.append((img, pos // iw, pos % iw))
    for img in (0, 100, 255):
        for r, c in ((0, 17), (55, 30), (23, 0), (40, 55), (0, 0), (0, 55), (55, 0), (55, 55)):
            pts.append((img, r, c))
    for _ in range(600):
        pts.append((int(rng.integers(bs)), int(rng.integers(ih)), int(rng.integers(iw))))
    pts = np.array(pts)
    want = np.empty((len(pts), oc))
    scale = np.empty((len(pts), oc))
    pad = {}
    for n_, (img, r, c) in enumerate(pts):
        if img not in pad:
            pad[img] = np.pad(xf[img], ((0, 0), (1, 1), (1, 1)))
        win = np.ascontiguousarray(pad[img][None, :, r:r + 3, c:c + 3])
        want[n_] = orc.conv2_naive_f64(win, wf, (0, 0), (1, 1), (1, 1))[0, :, 0, 0]
        scale[n_] = orc.conv2_naive_f64(np.abs(win), np.abs(wf), (0, 0), (1, 1), (1, 1))[0, :, 0, 0]
    k = ic * 9
    tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
    results = {}
    for alg in ("im2col", "direct"):
        fn = ag.conv2_im2col_forward if alg == "im2col" else ag.conv2_direct_forward
        y = fn(tx, tw, padding=(1, 1)).into_array()
        assert y.shape == (bs, oc, ih, iw)
        got = as_f32(np.ascontiguousarray(y[pts[:, 0], :, pts[:, 1], pts[:, 2]])).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(got - want) <= 1e-5 * np.sqrt(k) * scale), alg
        else:
            ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0**-126))) - 7)
            assert np.all(np.abs(got - want) <= ulp + 1e-2 * np.abs(want) + 8 * np.sqrt(k) * 2.0**-24 * scale), alg
        # nothing left unwritten: every output was produced by this launch
        assert np.isfinite(as_f32(y[::37].reshape(-1))).all()
        # bias + relu epilogue against the separate ops on this very result, on whole images
        yb = fn(tx, tw, padding=(1, 1), bias=tb, relu=True).into_array()
        for img in (0, 31, 32, 140, 255):
            flat = np.ascontiguousarray(y[img].reshape(oc, -1).T)
            ref = orc.relu(orc.bias_add_rows(flat, b)).T.reshape(oc, ih, iw)
            assert np.array_equal(yb[img], ref), (alg, img)
        results[alg] = y
        del yb
    # the two algorithms add the same products in different orders
    a_, d_ = as_f32(results["im2col"][::16]).astype(np.float64), as_f32(results["direct"][::16]).astype(np.float64)
    tol = (2e-5 * np.sqrt(k) if dtype == "f32" else 2.0**-6) * np.maximum(np.abs(a_), 1.0)
    assert np.all(np.abs(a_ - d_) <= tol)


def he(rng, shape, fan_in):  # Uniform(-a, a), a = sqrt(2/fan_in): layer.rs:345-349, :463-467
    a = np.sqrt(2.0 / fan_in)
    return rng.uniform(-a, a, shape).astype(np.float32)


def lenet_params(rng):
    return [he(rng, (6, 1, 5, 5), 25), he(rng, (16, 6, 5, 5), 150), he(rng, (256, 128), 256), he(rng, (128, 84), 128),
            he(rng, (84, 10), 84), he(rng, (10,), 84)]


def oracle_lenet_bf16(x, params):
    """The reference's DEVICE numerics for bf16 (f32 accumulate, one rounding per op), layer by layer."""
    w1, w2, wd1, wd2, wd3, b3 = params

    def conv(h, w):
        bs, ic, ih, iw = h.shape
        oc, _, fh, fw = w.shape
        cols = orc.im2col_conv2(h, (fh, fw))
        out = orc.gemm_bf16_f32acc(cols, w.reshape(oc, -1).T)
        oh, ow = ih - fh + 1, iw - fw + 1
        return np.ascontiguousarray(out.reshape(bs, oh, ow, oc).transpose(0, 3, 1, 2))

    h = orc.max_pool2(orc.relu(conv(x, w1)), (2, 2))
    h = orc.max_pool2(orc.relu(conv(h, w2)), (2, 2)).reshape(x.shape[0], 256)
    h = orc.relu(orc.gemm_bf16_f32acc(h, wd1))
    h = orc.relu(orc.gemm_bf16_f32acc(h, wd2))
    return orc.bias_add_rows(orc.gemm_bf16_f32acc(h, wd3), b3)


@pytest.mark.parametrize("bs", [1, 100, 1000])
def test_lenet5_forward_f32(ag, bs):
    rng = np.random.default_rng(23)
    params = lenet_params(rng)
    x = rng.uniform(0, 1, (bs, 1, 28, 28)).astype(np.float32)
    want = orc.lenet5_forward_f32(x, *params)
    model = ag.LeNet5.from_arrays(*params)
    tx = ag.Tensor.from_array(x)
    tol = 2e-4 * max(1.0, np.abs(want).max())  # six chained f32 layers, k up to 256
    for name, out in (("im2col", model.forward(tx, algorithm="im2col")), ("direct", model.forward(tx, algorithm="direct")),
                      ("fused", model.forward_fused(tx)), ("single", model.forward_single_launch(tx))):
        got = out.into_array()
        assert got.shape == (bs, 10)
        assert np.abs(got - want).max() <= tol, (name, np.abs(got - want).max())
    # graph-captured inference: several replays, each checked, with host work between them
    host = C.c_void_p()
    ag._ffi.check(ag.lib.agh_host_alloc(C.byref(host), bs * 10 * 4))
    logits = model.capture(tx, host.value)
    eager = model.forward_fused(tx).into_array()
    for i in range(4):
        ag._ffi.check(ag.lib.agh_memset(logits._ptr(), 0xFF, bs * 10 * 4))
        model.replay()
        ag._ffi.check(ag.lib.agh_sync())
        pinned = np.ctypeslib.as_array(C.cast(host.value, C.POINTER(C.c_float)), shape=(bs, 10)).copy()
        assert np.array_equal(pinned, eager), i
        assert np.array_equal(logits.into_array(), eager), i
    # single-launch kernel writing straight into pinned host memory
    single = model.forward_single_launch(tx).into_array()
    for i in range(3):
        C.memset(host.value, 0xFF, bs * 10 * 4)
        model.forward_single_launch(tx, host.value)
        ag._ffi.check(ag.lib.agh_sync())
        pinned = np.ctypeslib.as_array(C.cast(host.value, C.POINTER(C.c_float)), shape=(bs, 10)).copy()
        assert np.array_equal(pinned, single), i
    del model
    ag._ffi.check(ag.lib.agh_host_free(host))


@pytest.mark.parametrize("bs", [1, 100])
def test_lenet5_forward_bf16(ag, bs):
    rng = np.random.default_rng(24)
    params = [orc.f32_to_bf16(p) for p in lenet_params(rng)]
    x = orc.f32_to_bf16(rng.uniform(0, 1, (bs, 1, 28, 28)).astype(np.float32))
    want = orc.bf16_to_f32(oracle_lenet_bf16(x, params)).astype(np.float64)
    model = ag.LeNet5.from_arrays(*params)
    tx = ag.Tensor.from_array(x)
    for name, out in (("im2col", model.forward(tx, algorithm="im2col")), ("fused", model.forward_fused(tx)),
                      ("single", model.forward_single_launch(tx))):
        got = orc.bf16_to_f32(out.into_array()).astype(np.float64)
        # every layer may differ from the oracle by one bf16 rounding; six layers compound
        assert np.abs(got - want).max() <= 0.05 * max(1.0, np.abs(want).max()), (name, np.abs(got - want).max())
        assert np.mean(np.abs(got - want)) <= 0.01 * max(1.0, np.abs(want).max()), name


def test_random_geometry_im2col_col2im_pool(ag):
    """200 seeded random geometries (filter 1..5 per axis, padding 0..2, stride 1..3, dilation 1..2, windows 1..3 with
    equal or other strides, inputs up to 39 x 39, both element types, a third of the pooling inputs quantised so that
    windows hold ties): im2col, col2im on a random patch matrix of the same geometry, MaxPool2 forward and backward,
    each bit for bit against the oracle's host loops (src/tensor/ops.rs:842-1037, :1117-1264)."""
    from autograph_amd.tensor import Col2ImConv2Options, Im2ColConv2Options, MaxPool2Options
    rng = np.random.default_rng(2718)

    def rnd(shape, dt):
        x = rng.standard_normal(shape).astype(np.float32)
        if rng.random() < 0.3:
            x = np.round(x * 2) / 2
        return to_dtype(x, dt)

    done = 0
    for _ in range(200):
        dt = "bf16" if rng.random() < 0.5 else "f32"
        bs, c = int(rng.integers(1, 5)), int(rng.integers(1, 20))
        ih, iw = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        if rng.random() < 0.4:
            iw = 8 * max(1, iw // 8)
        fh, fw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if rng.random() < 0.5:
            fw = fh
        pad = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
        st = (1, 1) if rng.random() < 0.6 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dl = (1, 1) if rng.random() < 0.7 else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        tag = (dt, bs, c, ih, iw, fh, fw, pad, st, dl)
        if ih + 2 * pad[0] >= dl[0] * (fh - 1) + 1 and iw + 2 * pad[1] >= dl[1] * (fw - 1) + 1:
            oh, ow = orc.conv_out(ih, fh, pad[0], st[0], dl[0]), orc.conv_out(iw, fw, pad[1], st[1], dl[1])
            x = rnd((bs, c, ih, iw), dt)
            got = ag.Tensor.from_array(x).im2col_conv2(Im2ColConv2Options((fh, fw), pad, st, dl)).into_array()
            assert np.array_equal(got, orc.im2col_conv2(x, (fh, fw), pad, st, dl)), tag
            o2h, o2w = orc.col2im_out(oh, fh, pad[0], st[0], dl[0]), orc.col2im_out(ow, fw, pad[1], st[1], dl[1])
            if o2h >= 1 and o2w >= 1:
                cols = rnd((bs * oh * ow, c * fh * fw), dt)
                got = ag.Tensor.from_array(cols).col2im_conv2(Col2ImConv2Options((oh, ow), (fh, fw), pad, st, dl)).into_array()
                assert np.array_equal(got, orc.col2im_conv2(cols, (oh, ow), (fh, fw), pad, st, dl)), tag
            done += 1
        kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        ps = (kh, kw) if rng.random() < 0.6 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        if ih >= kh and iw >= kw:
            x = rnd((bs, c, ih, iw), dt)
            want = orc.max_pool2(x, (kh, kw), ps)
            assert np.array_equal(ag.Tensor.from_array(x).max_pool2(MaxPool2Options((kh, kw), ps)).into_array(), want), (tag, kh, kw, ps)
            dy = rnd(want.shape, dt)
            tb = ag.Tensor.from_array(x)
            tb.max_pool2_backward(ag.Tensor.from_array(dy), MaxPool2Options((kh, kw), ps))
            assert np.array_equal(tb.into_array(), orc.max_pool2_backward(x, dy, (kh, kw), ps)), (tag, kh, kw, ps)
    assert done >= 150


def test_random_geometry_conv2_forward(ag):
    """80 seeded random convolutions, more than half of them shaped for the matrix-core kernel (16..64 input channels, 64
    or 128 output channels, rows of whole vectors, unit stride), the rest small with strides and dilations: both
    algorithms against the naive f64 convolution (f32: 1e-5 sqrt(K); bf16: 1 ulp + 1e-2 relative + a floor where the
    sum cancels), and bias + ReLU bit-identical to the separate ops on that very result (layer.rs:950-1005)."""
    rng = np.random.default_rng(31415)
    direct = 0
    for _ in range(80):
        dt = "bf16" if rng.random() < 0.5 else "f32"
        if rng.random() < 0.6:
            bs, ic, oc = int(rng.integers(1, 4)), 16 * int(rng.integers(1, 5)), 64 * int(rng.integers(1, 3))
            ih, iw = int(rng.integers(6, 40)), 8 * int(rng.integers(2, 6))
            st = dl = (1, 1)
        else:
            bs, ic, oc = int(rng.integers(1, 4)), int(rng.integers(1, 9)), int(rng.integers(1, 20))
            ih, iw = int(rng.integers(4, 30)), int(rng.integers(4, 30))
            st = (1, 1) if rng.random() < 0.6 else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
            dl = (1, 1) if rng.random() < 0.8 else (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        fh, fw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        pad = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
        if ih + 2 * pad[0] < dl[0] * (fh - 1) + 1 or iw + 2 * pad[1] < dl[1] * (fw - 1) + 1:
            continue
        x = to_dtype(rng.standard_normal((bs, ic, ih, iw)), dt)
        w = to_dtype(rng.standard_normal((oc, ic, fh, fw)) * np.sqrt(2.0 / (ic * fh * fw)), dt)
        b = to_dtype(rng.standard_normal(oc), dt)
        want = orc.conv2_naive_f64(as_f32(x), as_f32(w), pad, st, dl)
        tag = (dt, bs, ic, ih, iw, oc, fh, fw, pad, st, dl)
        tx, tw, tb = ag.Tensor.from_array(x), ag.Tensor.from_array(w), ag.Tensor.from_array(b)
        scale = max(np.abs(want).max(), 1e-6)
        for alg in ("im2col", "direct"):
            fn = ag.conv2_im2col_forward if alg == "im2col" else ag.conv2_direct_forward
            try:
                y = fn(tx, tw, padding=pad, stride=st, dilation=dl).into_array()
                yb = fn(tx, tw, padding=pad, stride=st, dilation=dl, bias=tb, relu=True).into_array()
            except ag.AghError as e:
                assert alg == "direct" and e.code == -4, (alg, tag)   # the layer does not fit the direct kernels
                continue
            direct += alg == "direct"
            yf = as_f32(y).astype(np.float64)
            if dt == "f32":
                assert np.abs(yf - want).max() <= 1e-5 * np.sqrt(ic * fh * fw) * scale, (alg, tag)
                assert np.array_equal(yb, np.maximum(y + b[None, :, None, None], 0.0)), (alg, tag)
            else:
                assert np.all(np.abs(yf - want) <= 2.0**-7 * np.abs(want) + 1e-2 * np.abs(want) + 2e-3 * scale), (alg, tag)
                s1 = orc.f32_to_bf16(as_f32(y) + as_f32(b)[None, :, None, None])
                assert np.array_equal(as_f32(yb), np.maximum(as_f32(s1), 0.0)), (alg, tag)
    assert direct >= 30
