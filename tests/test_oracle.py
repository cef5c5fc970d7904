"""Pins the CPU oracle before anything is compared with it (runs without a GPU).

Each oracle function is checked against something that is NOT a retyping of its own
loop: a library routine it must reduce to (torch unfold / fold / max_pool2d / conv2d,
numpy float64 matmul), closed forms and invariants, and the generators the reference's
own tests use (integer ramps and cycles, tests/integration_tests.rs:291-305,
:1499-1628), on which every float sum is exact.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc
from refgrid import DOT_SIZES, POOL_SHAPES, cases, conv_options, input_shapes, BATCH_IN_OUT


def bf16_bits_torch(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


# ---------------------------------------------------------------- bf16 ----
def test_bf16_roundtrip_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    f = orc.bf16_to_f32(bits)
    back = orc.f32_to_bf16(f)
    nan = (bits & 0x7FFF) > 0x7F80
    assert np.array_equal(back[~nan], bits[~nan])
    # NaNs come back quiet with the payload kept
    assert np.array_equal(back[nan], bits[nan] | 0x40)
    # widening is a plain shift for every non-NaN pattern
    assert np.array_equal(f[~nan].view(np.uint32), bits[~nan].astype(np.uint32) << 16)


def test_bf16_rne_matches_torch_and_closed_form():
    rng = np.random.default_rng(0)
    # every exponent, random mantissas, plus exact ties and their neighbours
    u = rng.integers(0, 2**32, size=400000, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 2**16, size=20000, dtype=np.uint32) << 16) | 0x8000
    u = np.concatenate([u, ties, ties + 1, ties - 1, np.array([0, 0x80000000, 0x7F7FFFFF, 0x7F800000, 0xFF800000, 0x00000001, 0x00008000, 0x00018000], dtype=np.uint32)])
    f = u.view(np.float32)
    finite = ~np.isnan(f)
    got = orc.f32_to_bf16(f)
    assert np.array_equal(got[finite], bf16_bits_torch(f)[finite])
    # closed form: nearest representable, ties to even, computed in integer arithmetic
    lo = (u >> 16).astype(np.uint32)
    rem = u & 0xFFFF
    up = (rem > 0x8000) | ((rem == 0x8000) & ((lo & 1) == 1))
    want = (lo + up).astype(np.uint16)
    assert np.array_equal(got[finite], want[finite])
    assert np.all((got[~finite] & 0x7FC0) == 0x7FC0)


# -------------------------------------------------------------- shapes ----
def test_shape_formulas_against_torch():
    for f, p, s, d in conv_options():
        for ih, iw in input_shapes(f, p, s, d):
            y = F.conv2d(torch.zeros(1, 1, ih, iw), torch.zeros(1, 1, *f), padding=p, stride=s, dilation=d)
            oh, ow = orc.conv_out(ih, f[0], p[0], s[0], d[0]), orc.conv_out(iw, f[1], p[1], s[1], d[1])
            assert (oh, ow) == tuple(y.shape[2:])
            # col2im's output formula inverts it whenever the stride divides evenly
            if (ih + 2 * p[0] - d[0] * (f[0] - 1) - 1) % s[0] == 0:
                assert orc.col2im_out(oh, f[0], p[0], s[0], d[0]) == ih
    for i, x, s in [(4, 2, 2), (24, 2, 2), (7, 3, 2), (9, 3, 1), (5, 2, 3)]:
        assert orc.pool_out(i, x, s) == F.max_pool2d(torch.zeros(1, 1, i, i), x, s).shape[-1]


# -------------------------------------------------------------- im2col ----
def torch_im2col(x, f, p, s, d):
    bs, c = x.shape[:2]
    u = F.unfold(torch.from_numpy(x), f, dilation=d, padding=p, stride=s)  # [bs, c*fh*fw, L]
    return u.transpose(1, 2).reshape(-1, c * f[0] * f[1]).numpy()


def test_im2col_reference_grid_vs_unfold():
    n = 0
    for bs, c, ih, iw, f, p, s, d in cases():
        x = np.arange(1, bs * c * ih * iw + 1, dtype=np.float32).reshape(bs, c, ih, iw)  # ramp, :1505
        y = orc.im2col_conv2(x, f, p, s, d)
        assert np.array_equal(y, torch_im2col(x, f, p, s, d)), (bs, c, ih, iw, f, p, s, d)
        # 16-bit elements move the same way
        xb = orc.f32_to_bf16(x)
        assert np.array_equal(orc.im2col_conv2(xb, f, p, s, d), orc.f32_to_bf16(y))
        n += 1
    assert n > 1000


def test_im2col_mixed_options_random():
    rng = np.random.default_rng(1)
    for (bs, c, ih, iw, f, p, s, d) in [(2, 3, 9, 11, (3, 2), (1, 2), (2, 1), (1, 2)), (1, 5, 14, 9, (5, 3), (2, 0), (3, 2), (2, 1)), (3, 2, 6, 6, (2, 2), (0, 0), (2, 2), (1, 1))]:
        x = rng.standard_normal((bs, c, ih, iw)).astype(np.float32)
        assert np.array_equal(orc.im2col_conv2(x, f, p, s, d).view(np.uint32), torch_im2col(x, f, p, s, d).view(np.uint32))


# -------------------------------------------------------------- col2im ----
def torch_col2im(cols, bs, c, out_hw, f, p, s, d):
    L = cols.shape[0] // bs
    t = torch.from_numpy(cols.astype(np.float64)).reshape(bs, L, c * f[0] * f[1]).transpose(1, 2)
    return F.fold(t, out_hw, f, dilation=d, padding=p, stride=s).numpy()


def test_col2im_reference_grid_exact_integers():
    for bs, c, ih, iw, f, p, s, d in cases():
        oh, ow = orc.conv_out(ih, f[0], p[0], s[0], d[0]), orc.conv_out(iw, f[1], p[1], s[1], d[1])
        rows, cols = bs * oh * ow, c * f[0] * f[1]
        dy = np.arange(1, rows * cols + 1, dtype=np.float32).reshape(rows, cols)  # ramp, :1535-1538
        if dy.max() * f[0] * f[1] >= 2**24:
            continue
        dx = orc.col2im_conv2(dy, (oh, ow), f, p, s, d)
        out_hw = (orc.col2im_out(oh, f[0], p[0], s[0], d[0]), orc.col2im_out(ow, f[1], p[1], s[1], d[1]))
        assert dx.shape == (bs, c) + out_hw
        want = torch_col2im(dy, bs, c, out_hw, f, p, s, d)
        assert np.array_equal(dx.astype(np.float64), want), (bs, c, ih, iw, f, p, s, d)


def test_col2im_of_ones_counts_windows():
    # col2im(im2col(1)) = how many patches cover each pixel
    for (ih, iw, f, p, s, d) in [(7, 9, (3, 3), (1, 1), (1, 1), (1, 1)), (8, 8, (2, 2), (0, 0), (2, 2), (1, 1)), (9, 7, (3, 2), (0, 1), (2, 1), (1, 2))]:
        ones = np.ones((2, 3, ih, iw), dtype=np.float32)
        cols = orc.im2col_conv2(ones, f, p, s, d)
        oh, ow = orc.conv_out(ih, f[0], p[0], s[0], d[0]), orc.conv_out(iw, f[1], p[1], s[1], d[1])
        cnt = orc.col2im_conv2(cols, (oh, ow), f, p, s, d)
        want = torch_col2im(cols, 2, 3, cnt.shape[2:], f, p, s, d)
        assert np.array_equal(cnt, want)
        # bf16 accumulates the same small integers exactly
        cntb = orc.col2im_conv2(orc.f32_to_bf16(cols), (oh, ow), f, p, s, d)
        assert np.array_equal(orc.bf16_to_f32(cntb), cnt)


def test_col2im_bf16_rounds_after_every_add_in_host_order():
    # One output pixel, three contributions a, b, c chosen so that
    # rn(rn(a+b)+c) != rn(a+(b+c)) != rn_f32sum: 256 + 1 + 1 in bf16 (8 significant bits).
    # 1x3 filter over a 1x3 grid, padding 1: the centre output pixel w=1 receives
    # (wid=0,fj=2), (wid=1,fj=1), (wid=2,fj=0) in that order (wid ascending).
    f, p = (1, 3), (0, 1)
    cols = np.zeros((3, 3), dtype=np.float32)
    cols[0, 2], cols[1, 1], cols[2, 0] = 256.0, 1.0, 1.0
    y = orc.bf16_to_f32(orc.col2im_conv2(orc.f32_to_bf16(cols), (1, 3), f, p))
    assert y.shape == (1, 1, 1, 3)
    assert y[0, 0, 0, 1] == 256.0  # (256+1 -> 256) + 1 -> 256 ; an f32 accumulator would give 258
    cols[0, 2], cols[1, 1], cols[2, 0] = 1.0, 1.0, 256.0
    y = orc.bf16_to_f32(orc.col2im_conv2(orc.f32_to_bf16(cols), (1, 3), f, p))
    assert y[0, 0, 0, 1] == 258.0  # (1+1) + 256 is exact
    # f32 path keeps f32 sums
    y32 = orc.col2im_conv2(cols, (1, 3), f, p)
    assert y32[0, 0, 0, 1] == 258.0


def test_col2im_f32_order_is_hid_then_wid():
    # 3 values whose f32 sum depends on the order: big, -big, small
    big, small = np.float32(2**25), np.float32(1.0)
    f, p = (3, 1), (1, 0)  # vertical 3-tap: centre pixel h=1 gets hid=0 (fi=2), hid=1 (fi=1), hid=2 (fi=0)
    cols = np.zeros((3, 3), dtype=np.float32)
    cols[0, 2], cols[1, 1], cols[2, 0] = small, big, -big
    y = orc.col2im_conv2(cols, (3, 1), f, p)
    assert y[0, 0, 1, 0] == 0.0  # ((0+1)+2^25)-2^25 = 0
    cols[0, 2], cols[1, 1], cols[2, 0] = big, -big, small
    y = orc.col2im_conv2(cols, (3, 1), f, p)
    assert y[0, 0, 1, 0] == 1.0


# ------------------------------------------------------------ max pool ----
def cyc(shape, dtype=np.float32):
    n = int(np.prod(shape))
    return (np.arange(n) % 10).astype(dtype).reshape(shape)  # (0..10).cycle(), :1556-1560


def test_max_pool2_reference_shapes_vs_torch():
    for shape in POOL_SHAPES:
        x = cyc(shape)
        y = orc.max_pool2(x, (2, 2))
        want, idx = F.max_pool2d(torch.from_numpy(x), 2, 2, return_indices=True)
        assert np.array_equal(y, want.numpy())
        dy = np.arange(y.size, dtype=np.float32).reshape(y.shape)  # 0..len ramp, :1605-1608
        dx = orc.max_pool2_backward(x, dy, (2, 2))
        # the cycling data contains ties inside windows; the first maximum in row-major
        # window order must win, which is what torch reports as the index
        want_dx = np.zeros(x.size, dtype=np.float32).reshape(shape[0] * shape[1], -1)
        flat_idx = idx.numpy().reshape(shape[0] * shape[1], -1)
        for pl in range(want_dx.shape[0]):
            want_dx[pl, flat_idx[pl]] = dy.reshape(shape[0] * shape[1], -1)[pl]
        assert np.array_equal(dx, want_dx.reshape(shape))
        yb = orc.max_pool2(orc.f32_to_bf16(x), (2, 2))
        assert np.array_equal(orc.bf16_to_f32(yb), y)
        dxb = orc.max_pool2_backward(orc.f32_to_bf16(x), orc.f32_to_bf16(dy), (2, 2))
        assert np.array_equal(orc.bf16_to_f32(dxb), orc.bf16_to_f32(orc.f32_to_bf16(dx)))


def test_max_pool2_first_max_wins_on_ties():
    x = np.array([[[[5, 5], [5, 5]]]], dtype=np.float32)
    dx = orc.max_pool2_backward(x, np.array([[[[7.0]]]], dtype=np.float32), (2, 2))
    assert np.array_equal(dx, np.array([[[[7, 0], [0, 0]]]], dtype=np.float32))
    x = np.array([[[[1, 9], [9, 3]]]], dtype=np.float32)
    dx = orc.max_pool2_backward(x, np.array([[[[2.0]]]], dtype=np.float32), (2, 2))
    assert np.array_equal(dx, np.array([[[[0, 2], [0, 0]]]], dtype=np.float32))


def test_max_pool2_special_values():
    nan = np.float32(np.nan)
    # leading NaN sticks (nothing is > NaN); a later NaN never replaces
    x = np.array([[[[nan, 3], [4, 5]]]], dtype=np.float32)
    assert np.isnan(orc.max_pool2(x, (2, 2))[0, 0, 0, 0])
    x = np.array([[[[1, nan], [4, 2]]]], dtype=np.float32)
    assert orc.max_pool2(x, (2, 2))[0, 0, 0, 0] == 4
    # -0 first, +0 later: +0 > -0 is false, so -0 is kept bit for bit
    x = np.array([[[[-0.0, 0.0], [0.0, -0.0]]]], dtype=np.float32)
    assert orc.max_pool2(x, (2, 2)).view(np.uint32)[0, 0, 0, 0] == 0x80000000
    xb = orc.f32_to_bf16(x)
    assert orc.max_pool2(xb, (2, 2))[0, 0, 0, 0] == 0x8000
    # backward: 0 + (-0) = +0
    dx = orc.max_pool2_backward(np.ones((1, 1, 2, 2), np.float32), np.array([[[[-0.0]]]], np.float32), (2, 2))
    assert dx.view(np.uint32)[0, 0, 0, 0] == 0


def test_max_pool2_general_windows_vs_torch_and_uncovered_cells():
    rng = np.random.default_rng(3)
    for (shape, size, st) in [((2, 3, 7, 9), (3, 2), (3, 2)), ((1, 2, 11, 10), (2, 3), (4, 5)), ((2, 2, 9, 9), (3, 3), (2, 2)), ((1, 1, 8, 8), (3, 3), (1, 1))]:
        x = rng.permutation(int(np.prod(shape))).astype(np.float32).reshape(shape)  # all distinct
        y = orc.max_pool2(x, size, st)
        want = F.max_pool2d(torch.from_numpy(x), size, st)
        assert np.array_equal(y, want.numpy())
    # stride > window: cells between windows keep their x value after backward
    x = rng.permutation(2 * 7 * 7).astype(np.float32).reshape(1, 2, 7, 7) + 1
    dy = rng.standard_normal((1, 2, 2, 2)).astype(np.float32)
    dx = orc.max_pool2_backward(x, dy, (2, 2), (4, 4))
    covered = np.zeros((7, 7), bool)
    for h0 in (0, 4):
        for w0 in (0, 4):
            covered[h0:h0 + 2, w0:w0 + 2] = True
    assert np.array_equal(dx[..., ~covered], x[..., ~covered])
    _, idx = F.max_pool2d(torch.from_numpy(x), 2, 4, return_indices=True)
    want = np.zeros((2, 49), np.float32)
    for pl in range(2):
        want[pl, idx.numpy().reshape(2, -1)[pl]] = dy.reshape(2, -1)[pl]
    assert np.array_equal(dx[..., covered], want.reshape(1, 2, 7, 7)[..., covered])


def test_max_pool2_backward_overlapping_windows_is_sequential():
    # 1x3 input, window 1x2 stride 1: window 0 zeroes cells 0,1 and puts dy0 at its
    # argmax; window 1 then reads the UPDATED cell 1.
    x = np.array([[[[1.0, 5.0, 2.0]]]], dtype=np.float32)
    dy = np.array([[[[10.0, 1.0]]]], dtype=np.float32)
    dx = orc.max_pool2_backward(x, dy, (1, 2), (1, 1))
    # w0: argmax cell1 -> cells (0,10,2); w1 sees (10,2): argmax cell1, zero both, cell1 = 0+1
    assert np.array_equal(dx, np.array([[[[0.0, 1.0, 0.0]]]], dtype=np.float32))


# ---------------------------------------------------------- relu / bias ----
def test_relu_rules():
    x = (np.arange(-10, 10).astype(np.float32))  # (-10..10).cycle(), :1632-1636
    assert np.array_equal(orc.relu(x), np.maximum(x, 0))
    sp = np.array([-0.0, np.nan, np.inf, -np.inf, 1e-45], dtype=np.float32)
    r = orc.relu(sp)
    assert r.view(np.uint32)[0] == 0x80000000 and r[1] == 0 and r[2] == np.inf and r[3] == 0 and r[4] == sp[4]
    rb = orc.relu(orc.f32_to_bf16(sp))
    assert rb[0] == 0x8000 and rb[1] == 0 and rb[3] == 0
    dy = np.arange(20, dtype=np.float32)
    assert np.array_equal(orc.relu_backward(x, dy), np.where(x >= 0, dy, 0))


def test_bias_add():
    rng = np.random.default_rng(4)
    y = rng.standard_normal((5, 7)).astype(np.float32)
    b = rng.standard_normal(7).astype(np.float32)
    assert np.array_equal(orc.bias_add_rows(y, b), b[None, :] + y)
    yb, bb = orc.f32_to_bf16(y), orc.f32_to_bf16(b)
    want = orc.f32_to_bf16(orc.bf16_to_f32(bb)[None, :] + orc.bf16_to_f32(yb))
    assert np.array_equal(orc.bias_add_rows(yb, bb), want)


# ---------------------------------------------------------------- gemm ----
def gen_array(shape):  # values 1..9 cycling, integration_tests.rs:291-305
    n = shape[0] * shape[1]
    return ((np.arange(n) % 9) + 1).astype(np.float32).reshape(shape)


@pytest.mark.parametrize("n", DOT_SIZES)
def test_gemm_checkers_exact_on_reference_generator(n):
    for ta in (False, True):
        for tb in (False, True):
            a = gen_array((n, n))
            b = gen_array((n, n))
            av, bv = (a.T if ta else a), (b.T if tb else b)
            want = av.astype(np.float64) @ bv.astype(np.float64)
            assert np.array_equal(orc.gemm_f64acc(av, bv), want)
            assert np.array_equal(orc.gemm_f32_host(av, bv).astype(np.float64), want)
            ab, bb = orc.f32_to_bf16(a), orc.f32_to_bf16(b)
            abv, bbv = (ab.T if ta else ab), (bb.T if tb else bb)
            assert np.array_equal(orc.gemm_f64acc(abv, bbv), want)
            got = orc.bf16_to_f32(orc.gemm_bf16_f32acc(abv, bbv))
            assert np.array_equal(got, orc.bf16_to_f32(orc.f32_to_bf16(want.astype(np.float32))))
            if n <= 32:
                # host fold rounds every step: within the reference's own epsilon = k (:356-361)
                fold = orc.bf16_to_f32(orc.gemm_bf16_hostfold(abv, bbv))
                assert np.all(np.abs(fold - want) <= n * np.maximum(1, np.abs(want) * 2**-8 * n))


def test_gemm_strided_views_offsets_alpha_beta():
    rng = np.random.default_rng(5)
    big_a = rng.uniform(-1, 1, (40, 50)).astype(np.float32)
    big_b = rng.uniform(-1, 1, (60, 45)).astype(np.float32)
    a = big_a[3:36:2, 5:44:3]          # 17 x 13, strides (100, 3), offset
    b = big_b[40:1:-3, 44:10:-3]       # 13 x 12, negative row and column strides
    c = rng.uniform(-1, 1, (17, 12)).astype(np.float32)
    want = 0.5 * (a.astype(np.float64) @ b.astype(np.float64)) + 2.0 * c
    assert np.allclose(orc.gemm_f64acc(a, b, 0.5, 2.0, c), want, rtol=1e-14, atol=1e-14)
    got = orc.gemm_f32_host(a, b, 0.5, 2.0, c)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(13) * np.max(np.abs(want))
    # beta == 0 must not read C (NaN-poisoned C stays out of the result)
    poison = np.full((17, 12), np.nan, dtype=np.float32)
    assert np.isfinite(orc.gemm_f32_host(a, b, 1.0, 0.0, poison)).all()


def test_gemm_f32_host_blocking_edges_vs_float64():
    rng = np.random.default_rng(6)
    for (m, k, n) in [(1, 1, 1), (7, 300, 9), (65, 257, 1030), (130, 513, 17)]:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        want = a.astype(np.float64) @ b.astype(np.float64)
        for av, bv in [(a, b), (np.asfortranarray(a), b), (a, np.asfortranarray(b))]:
            got = orc.gemm_f32_host(av, bv, threads=3)
            assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(k) * max(1.0, np.max(np.abs(want)))


def test_gemm_bf16_f32acc_vs_float64():
    rng = np.random.default_rng(7)
    a = orc.f32_to_bf16(rng.normal(0, 0.02, (33, 200)).astype(np.float32))
    b = orc.f32_to_bf16(rng.normal(0, 0.02, (200, 29)).astype(np.float32))
    want = orc.bf16_to_f32(a).astype(np.float64) @ orc.bf16_to_f32(b).astype(np.float64)
    assert np.allclose(orc.gemm_f64acc(a, b), want, rtol=1e-13, atol=0)
    got = orc.bf16_to_f32(orc.gemm_bf16_f32acc(a, b)).astype(np.float64)
    ulp = np.abs(want) * 2.0**-7
    assert np.all(np.abs(got - want) <= ulp + 1e-2 * np.abs(want))


# ---------------------------------------------------------------- conv ----
def test_conv2_naive_vs_torch_conv2d_reference_generator():
    # x, w = (1..=10).cycle(), integration_tests.rs:1190-1207 ; all sums exact
    k = 0
    for f, p, s, d in conv_options():
        for ih, iw in list(input_shapes(f, p, s, d))[::5]:
            for bs, ic, oc in BATCH_IN_OUT[::3]:
                x = ((np.arange(bs * ic * ih * iw) % 10) + 1).astype(np.float32).reshape(bs, ic, ih, iw)
                w = ((np.arange(oc * ic * f[0] * f[1]) % 10) + 1).astype(np.float32).reshape(oc, ic, *f)
                y = orc.conv2_naive_f64(x, w, p, s, d)
                want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), padding=p, stride=s, dilation=d).numpy()
                assert np.array_equal(y, want)
                # conv2_im2col chain (layer.rs:950-1005) built from oracle parts equals it
                cols = orc.im2col_conv2(x, f, p, s, d)
                wm = w.reshape(oc, -1)
                om = orc.gemm_f64acc(cols, wm.T)
                oh, ow = y.shape[2:]
                assert np.array_equal(om.reshape(bs, oh, ow, oc).transpose(0, 3, 1, 2), want)
                k += 1
    assert k > 100


def test_lenet5_forward_vs_torch():
    rng = np.random.default_rng(8)
    bs = 6
    x = rng.uniform(0, 1, (bs, 1, 28, 28)).astype(np.float32)

    def he(shape, fan_in):  # Uniform(-a, a), a = sqrt(2/fan_in): layer.rs:345-349, :463-467
        a = np.sqrt(2.0 / fan_in)
        return rng.uniform(-a, a, shape).astype(np.float32)

    w1, w2 = he((6, 1, 5, 5), 25), he((16, 6, 5, 5), 150)
    wd1, wd2, wd3, b3 = he((256, 128), 256), he((128, 84), 128), he((84, 10), 84), he((10,), 84)
    got = orc.lenet5_forward_f32(x, w1, w2, wd1, wd2, wd3, b3)
    t = torch.from_numpy
    h = F.max_pool2d(F.relu(F.conv2d(t(x).double(), t(w1).double())), 2)
    h = F.max_pool2d(F.relu(F.conv2d(h, t(w2).double())), 2).flatten(1)
    h = F.relu(h @ t(wd1).double())
    h = F.relu(h @ t(wd2).double())
    want = (h @ t(wd3).double() + t(b3).double()).numpy()
    assert np.max(np.abs(got - want)) < 1e-4 * max(1.0, np.max(np.abs(want)))
    got_direct = orc.lenet5_forward_f32(x, w1, w2, wd1, wd2, wd3, b3, direct=True)
    assert np.max(np.abs(got_direct - want)) < 1e-4 * max(1.0, np.max(np.abs(want)))


def test_conv2_direct_host_vs_torch():
    rng = np.random.default_rng(9)
    for (bs, ic, ih, iw, oc, f) in [(3, 1, 28, 28, 6, (5, 5)), (2, 6, 12, 12, 16, (5, 5)), (1, 3, 9, 7, 4, (3, 2))]:
        x = rng.standard_normal((bs, ic, ih, iw)).astype(np.float32)
        w = rng.standard_normal((oc, ic) + f).astype(np.float32)
        want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double()).numpy()
        got = orc.conv2_direct_f32(x, w)
        assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(ic * f[0] * f[1]) * np.max(np.abs(want))


def test_conv2_direct_packed_host_vs_torch_and_exact_on_integers():
    """The packed, register-tiled restatement of conv2_direct_host_f32 (conv_direct.rs:760-946) against torch's
    float64 convolution and, bit for bit, on small-integer data (every sum exact).  Shapes cover: ic == 1 (unpacked
    input, TCX = 1) and ic > 1 (TCX = 8) with ic below, equal to and above a multiple of 8; oc below 8, a multiple
    of 8 and above 32 (more than one chunk of four 8-channel blocks, a ragged last chunk); output rows shorter than
    the column tile, equal to it and with a ragged last tile; one thread and many (images dealt round robin)."""
    rng = np.random.default_rng(91)
    shapes = [(3, 1, 28, 28, 6, (5, 5)), (5, 6, 12, 12, 16, (5, 5)), (2, 3, 9, 7, 4, (3, 2)), (2, 8, 6, 6, 8, (1, 1)),
              (3, 11, 10, 13, 40, (3, 3)), (1, 17, 5, 9, 33, (2, 3)), (4, 1, 7, 3, 9, (2, 2)), (2, 16, 8, 11, 24, (3, 5)),
              (7, 2, 6, 23, 20, (3, 3))]
    for (bs, ic, ih, iw, oc, f) in shapes:
        x = rng.standard_normal((bs, ic, ih, iw)).astype(np.float32)
        w = rng.standard_normal((oc, ic) + f).astype(np.float32)
        want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double()).numpy()
        for threads in (1, 0):
            got = orc.conv2_direct_packed_f32(x, w, threads=threads)
            assert got.shape == want.shape
            assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(ic * f[0] * f[1]) * np.max(np.abs(want)), (bs, ic, oc, f)
        xi = rng.integers(-4, 5, (bs, ic, ih, iw)).astype(np.float32)
        wi = rng.integers(-4, 5, (oc, ic) + f).astype(np.float32)
        exact = F.conv2d(torch.from_numpy(xi).double(), torch.from_numpy(wi).double()).numpy()
        assert np.array_equal(orc.conv2_direct_packed_f32(xi, wi).astype(np.float64), exact), (bs, ic, oc, f)
    # and the LeNet5 forward pass built on it agrees with the im2col + sgemm chain
    x = rng.uniform(0, 1, (20, 1, 28, 28)).astype(np.float32)
    params = [rng.standard_normal(s).astype(np.float32) * 0.1 for s in ((6, 1, 5, 5), (16, 6, 5, 5), (256, 128), (128, 84), (84, 10), (10,))]
    a = orc.lenet5_forward_f32(x, *params, direct="packed")
    b = orc.lenet5_forward_f32(x, *params)
    assert np.max(np.abs(a - b)) <= 2e-5 * np.max(np.abs(b))


# ------------------------------------------------------------ training tail ----
def tbf(x):
    """numpy uint16 bf16 bits -> torch.bfloat16 tensor."""
    return torch.from_numpy(np.ascontiguousarray(x).view(np.int16)).view(torch.bfloat16)


def tbits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_assign4_strided_views_vs_numpy():
    rng = np.random.default_rng(31)
    base = rng.integers(0, 2**16, (5, 6, 7, 8)).astype(np.uint16)
    views = [base.transpose(0, 2, 3, 1), base.transpose(3, 2, 1, 0), base[::2, ::-1, 1:6, ::3], base[:, 2],
             base[1, :, 3], np.broadcast_to(base[0, 0, 0], (4, 8)), base.astype(np.float32).transpose(0, 3, 1, 2)]
    for v in views:
        got = orc.to_standard_layout(v)
        assert got.flags["C_CONTIGUOUS"] and np.array_equal(got, np.ascontiguousarray(v))


def test_scaled_add_vs_torch_per_op_rounding():
    """bf16: the product and the sum round separately (torch.bfloat16 elementwise ops do exactly that)."""
    rng = np.random.default_rng(32)
    y = orc.f32_to_bf16(rng.standard_normal(5000).astype(np.float32))
    x = orc.f32_to_bf16(rng.standard_normal(5000).astype(np.float32) * 3)
    alpha = -0.01
    a_t = torch.tensor(alpha, dtype=torch.float32).to(torch.bfloat16)
    want = tbits(a_t * tbf(x) + tbf(y))
    assert np.array_equal(orc.scaled_add(y, alpha, x), want)
    # a fused multiply-add would differ somewhere on this much data: the check can tell the two apart
    fused = orc.f32_to_bf16(orc.bf16_to_f32(y) + float(a_t) * orc.bf16_to_f32(x))
    assert not np.array_equal(fused, want)
    yf, xf = rng.standard_normal(1000).astype(np.float32), rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(orc.scaled_add(yf, 0.3, xf), (np.float32(0.3) * xf) + yf)


def test_scaled_add_strided_vs_torch_on_views():
    """`scaled_add` on views (src/tensor/ops.rs:192-204, :257-318): torch evaluates `y_view += a * x` on strided and
    broadcast operands with one bf16 rounding per operation; the oracle must leave every element outside the
    destination view untouched and agree bit for bit inside it."""
    rng = np.random.default_rng(132)
    a_t = torch.tensor(0.3, dtype=torch.float32).to(torch.bfloat16)

    def run(ybase, yview, x):
        """yview(array) picks the destination view out of a base array; x is broadcast against it."""
        for bf in (True, False):
            yb = orc.f32_to_bf16(ybase) if bf else ybase.copy()
            xv = orc.f32_to_bf16(x) if bf else x.copy()
            want = yb.copy()
            dst = yview(want)
            if bf:  # torch rounds the product and the sum separately; done on contiguous copies of the view
                prod = a_t * tbf(np.ascontiguousarray(np.broadcast_to(xv, dst.shape)))
                dst[...] = tbits(prod + tbf(np.ascontiguousarray(dst)))
            else:
                dst[...] = (np.float32(0.3) * np.broadcast_to(xv, dst.shape)).astype(np.float32) + dst
            orc.scaled_add_strided(yview(yb), 0.3, xv)
            assert np.array_equal(yb, want)
            assert not np.array_equal(yb, orc.f32_to_bf16(ybase) if bf else ybase)

    base = rng.standard_normal((6, 10, 12)).astype(np.float32)
    run(base, lambda t: t, rng.standard_normal(12).astype(np.float32))                       # bias over the trailing axis
    run(base, lambda t: t[:, ::2, 1:9], rng.standard_normal((5, 8)).astype(np.float32))      # sliced destination
    run(base, lambda t: t.transpose(2, 1, 0), rng.standard_normal((1, 10, 1)).astype(np.float32))  # permuted destination
    run(base, lambda t: t[:, ::-1], rng.standard_normal((6, 1, 12)).astype(np.float32))      # negative stride
    run(base, lambda t: t, rng.standard_normal((1,)).astype(np.float32))                     # scalar broadcast
    # aliasing element for element: y += a * y
    yb = orc.f32_to_bf16(base)
    ty = tbf(yb).clone()
    ty.add_(a_t * ty.clone())
    got = yb.copy()
    orc.scaled_add_strided(got, 0.3, got)
    assert np.array_equal(got, tbits(ty))
    # the contiguous entry is the same operation
    x1 = orc.f32_to_bf16(rng.standard_normal(base.shape).astype(np.float32))
    got = yb.copy()
    orc.scaled_add_strided(got, -0.01, x1)
    assert np.array_equal(got, orc.scaled_add(yb, -0.01, x1))


def test_accuracy_reference_generator_and_rules():
    """accuracy_host (src/learn/criterion.rs:30-47).  On the reference test's data (tests/integration_tests.rs:767-793:
    rows are rotations of 0..classes starting at classes/2 + 1, targets cycle 0..classes) every row is a permutation,
    so a row counts exactly when its target holds the row's maximum classes - 1: a closed form, not the oracle's loop."""
    for bs, classes in [(1, 8), (31, 16), (1000, 100)]:
        flat = np.resize(np.arange(classes), bs * classes + classes // 2 + 1)[classes // 2 + 1:][: bs * classes]
        x = flat.reshape(bs, classes).astype(np.float32)
        t = (np.arange(bs) % classes).astype(np.uint8)
        want = int(np.sum(x[np.arange(bs), t] == classes - 1))
        assert orc.accuracy(x, t) == want
        assert orc.accuracy(orc.f32_to_bf16(x), t) == want
    # ties, NaNs and out-of-range targets do not count; strictly greater does
    x = np.array([[1, 3, 2], [3, 3, 1], [np.nan, 1, 0], [0, np.nan, 5], [2, 1, 0], [-0.0, 0.0, -1]], dtype=np.float32)
    t = np.array([1, 0, 0, 2, 7, 0], dtype=np.uint8)
    assert orc.accuracy(x, t) == 1
    assert orc.accuracy(orc.f32_to_bf16(x), t) == 1
    # against argmax with a uniqueness check on random data with many ties
    rng = np.random.default_rng(133)
    x = rng.integers(0, 4, (500, 6)).astype(np.float32)
    t = rng.integers(0, 6, 500).astype(np.uint8)
    top = x.max(axis=1)
    want = int(np.sum((x[np.arange(500), t] == top) & ((x == top[:, None]).sum(axis=1) == 1)))
    assert orc.accuracy(x, t) == want


def test_sgd_momentum_vs_closed_form():
    rng = np.random.default_rng(33)
    w, dw, v = (rng.standard_normal(3000).astype(np.float32) for _ in range(3))
    lr, m = np.float32(0.01), np.float32(0.9)
    vn = m * v + dw
    w2, v2 = orc.sgd_momentum(w, dw, lr, m, v)
    assert np.array_equal(v2, vn) and np.array_equal(w2, w - lr * vn)
    wb, dwb, vb = orc.f32_to_bf16(w), orc.f32_to_bf16(dw), orc.f32_to_bf16(v)
    vnf = m * orc.bf16_to_f32(vb) + orc.bf16_to_f32(dwb)
    w2, v2 = orc.sgd_momentum(wb, dwb, lr, m, vb)
    # the weight uses the UNrounded new velocity (optimizer.rs:509-512 runs in f32, casts at the end)
    assert np.array_equal(v2, bf16_bits_torch(vnf)) and np.array_equal(w2, bf16_bits_torch(orc.bf16_to_f32(wb) - lr * vnf))


def test_sum_axis0_is_sequential_in_element_type():
    # 256 + 1 + 1 + ... in bf16 stays 256 when added one by one (ulp(256) = 2); any pairwise order gives more
    x = orc.f32_to_bf16(np.array([[256.0, 1.0]] + [[1.0, 1.0]] * 64, dtype=np.float32))
    assert orc.bf16_to_f32(orc.sum_axis0(x)).tolist() == [256.0, 65.0]
    rng = np.random.default_rng(34)
    xb = orc.f32_to_bf16(rng.standard_normal((100, 10)).astype(np.float32))
    acc = torch.zeros(10, dtype=torch.bfloat16)
    for row in tbf(xb):
        acc = acc + row
    assert np.array_equal(orc.sum_axis0(xb), tbits(acc))
    xf = rng.standard_normal((50, 7)).astype(np.float32)
    want = np.zeros(7, dtype=np.float32)
    for row in xf:
        want = want + row
    assert np.array_equal(orc.sum_axis0(xf), want)


def test_cross_entropy_vs_torch():
    rng = np.random.default_rng(35)
    for bs, classes in [(100, 10), (7, 3), (1, 5)]:
        x = (rng.standard_normal((bs, classes)) * 3).astype(np.float32)
        t = rng.integers(0, classes, bs).astype(np.uint8)
        xt = torch.from_numpy(x).double().requires_grad_(True)
        loss = F.cross_entropy(xt, torch.from_numpy(t).long(), reduction="sum")
        (loss / bs).backward()
        assert abs(orc.cross_entropy_loss(x, t) - loss.item()) <= 2e-6 * max(1.0, abs(loss.item()))
        assert np.allclose(orc.cross_entropy_backward(x, t), xt.grad.numpy(), rtol=1e-5, atol=1e-8)
        xb = orc.f32_to_bf16(x)
        xbt = torch.from_numpy(orc.bf16_to_f32(xb)).double().requires_grad_(True)
        lossb = F.cross_entropy(xbt, torch.from_numpy(t).long(), reduction="sum")
        (lossb / bs).backward()
        assert abs(orc.cross_entropy_loss(xb, t) - lossb.item()) <= 2e-6 * max(1.0, abs(lossb.item()))
        gb = orc.bf16_to_f32(orc.cross_entropy_backward(xb, t)).astype(np.float64)
        assert np.all(np.abs(gb - xbt.grad.numpy()) <= 2.0**-8 * np.abs(xbt.grad.numpy()) + 1e-12)
    # huge logits: the max is subtracted before exp
    x = np.array([[1000.0, 999.0, -1000.0]], dtype=np.float32)
    assert abs(orc.cross_entropy_loss(x, np.array([1], dtype=np.uint8)) - (np.log1p(np.exp(-1.0)) + 1.0)) < 1e-6


def lenet_params_np(rng):
    def he(shape, fan_in):
        a = np.sqrt(2.0 / fan_in)
        return rng.uniform(-a, a, shape).astype(np.float32)
    return [he((6, 1, 5, 5), 25), he((16, 6, 5, 5), 150), he((256, 128), 256), he((128, 84), 128), he((84, 10), 84), he((10,), 84)]


def torch_lenet_grads(x, t, params):
    p = [torch.from_numpy(a).double().requires_grad_(True) for a in params]
    h = F.max_pool2d(F.relu(F.conv2d(torch.from_numpy(x).double(), p[0])), 2)
    h = F.max_pool2d(F.relu(F.conv2d(h, p[1])), 2).reshape(x.shape[0], 256)
    logits = F.relu(F.relu(h @ p[2]) @ p[3]) @ p[4] + p[5]
    loss = F.cross_entropy(logits, torch.from_numpy(t).long(), reduction="sum")
    (loss / x.shape[0]).backward()
    return loss.item(), [a.grad.numpy() for a in p]


def test_lenet5_train_step_f32_vs_torch_autograd():
    """Pins the whole backward chain (transposes, col2im geometry, pool/relu masks, bias sum, update sign)."""
    rng = np.random.default_rng(36)
    params = lenet_params_np(rng)
    x = rng.uniform(0, 1, (20, 1, 28, 28)).astype(np.float32)
    t = rng.integers(0, 10, 20).astype(np.uint8)
    loss, new_params, grads, _ = orc.lenet5_train_step(x, t, params, lr=0.01)
    want_loss, want_grads = torch_lenet_grads(x, t, params)
    assert abs(loss - want_loss) <= 1e-5 * abs(want_loss)
    for g, w, p, pn in zip(grads, want_grads, params, new_params):
        assert g.shape == w.shape
        assert np.abs(g - w).max() <= 2e-5 * max(1e-3, np.abs(w).max())
        assert np.array_equal(pn, (np.float32(-0.01) * g) + p)
    # momentum variant: first step from zero velocity
    _, p_m, _, v_m = orc.lenet5_train_step(x, t, params, lr=0.01, momentum=0.01)
    for g, p, pn, v in zip(grads, params, p_m, v_m):
        assert np.array_equal(v, g) and np.array_equal(pn, p - np.float32(0.01) * g)


def test_lenet5_train_step_bf16_close_to_f64_grads():
    rng = np.random.default_rng(37)
    params = [orc.f32_to_bf16(p) for p in lenet_params_np(rng)]
    x = orc.f32_to_bf16(rng.uniform(0, 1, (20, 1, 28, 28)).astype(np.float32))
    t = rng.integers(0, 10, 20).astype(np.uint8)
    loss, new_params, grads, _ = orc.lenet5_train_step(x, t, params, lr=0.01)
    want_loss, want_grads = torch_lenet_grads(orc.bf16_to_f32(x), t, [orc.bf16_to_f32(p) for p in params])
    assert abs(loss - want_loss) <= 2e-2 * abs(want_loss)
    for g, w in zip(grads, want_grads):
        gf = orc.bf16_to_f32(g).astype(np.float64)
        # bf16 activations and gradients round at every layer (and flip a few relu/pool decisions):
        # up to about a tenth of the largest entry on single elements, far less on average
        assert np.abs(gf - w).max() <= 0.12 * np.abs(w).max()
        assert np.abs(gf - w).mean() <= 0.02 * np.abs(w).max()
    for p, pn, g in zip(params, new_params, grads):
        assert np.array_equal(pn, orc.scaled_add(p, -0.01, g))
