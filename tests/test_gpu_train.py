"""GPU parity of the kernels a training step adds around the contraction path (strided copy,
scaled_add, SGD, axis-0 sum, cross-entropy) and of one whole LeNet5 training step
(benches/neural-network-benches/src/autograph_backend.rs:70-86) against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle as orc

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


def labels(ag, t):
    buf = ag.Buffer(t.size)
    ag._ffi.check(ag.lib.agh_memcpy_h2d(buf.ptr, t.ctypes.data, t.size))
    ag._ffi.check(ag.lib.agh_sync())
    return buf


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_assign_strided_views(ag, dtype):
    rng = np.random.default_rng(41)
    base = to_dtype(rng.standard_normal((5, 6, 7, 8)), dtype)
    t = ag.Tensor.from_array(base)
    for axes in [(0, 2, 3, 1), (0, 3, 1, 2), (3, 2, 1, 0), (1, 0, 3, 2)]:
        got = t.permuted_axes(axes).to_standard_layout().into_array()
        assert np.array_equal(got, np.ascontiguousarray(base.transpose(axes)))
    m = ag.Tensor.from_array(base.reshape(30, 56))
    assert np.array_equal(m.t().to_standard_layout().into_array(), np.ascontiguousarray(base.reshape(30, 56).T))
    assert np.array_equal(m.slice_rows(None, None, -2).to_standard_layout().into_array(), base.reshape(30, 56)[::-2])
    v = ag.Tensor.from_array(base[0, 0, 0])  # [8] broadcast over rows
    assert np.array_equal(v.broadcast((4, 8)).to_standard_layout().into_array(), np.broadcast_to(base[0, 0, 0], (4, 8)))
    # the conv backward's NCHW -> NHWC copy at LeNet5 size
    g = to_dtype(rng.standard_normal((100, 16, 8, 8)), dtype)
    got = ag.Tensor.from_array(g).permuted_axes((0, 2, 3, 1)).to_standard_layout().into_array()
    assert np.array_equal(got, orc.to_standard_layout(g.transpose(0, 2, 3, 1)))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_assign_large_transposing_copies(ag, dtype):
    """`to_standard_layout` of permuted views whose source and destination are contiguous along different axes
    (src/tensor/ops.rs:257-318, the NHWC <-> NCHW copies of layer.rs:1000-1004 and autograd.rs:396-445): these
    take the LDS-tiled path.  Bit-exact against the oracle's strided copy: whole and partial 64 x 64 tiles, the
    16-byte and the element-wise form (odd sizes, views at odd offsets), one and two batch dimensions,
    and the Conv2 activation of the benchmark list (256 x 128 x 56 x 56) in both directions."""
    rng = np.random.default_rng(44)
    cases = [((4, 64, 64), (0, 2, 1)), ((3, 128, 200), (0, 2, 1)), ((2, 3, 72, 40), (0, 1, 3, 2)), ((5, 17, 33), (0, 2, 1)),
             ((1, 100, 1000), (0, 2, 1)), ((2, 56, 56, 128), (0, 3, 1, 2)), ((2, 128, 56, 56), (0, 2, 3, 1)),
             ((7, 19, 23, 16), (0, 3, 1, 2)), ((300, 70), (1, 0)), ((4, 5, 96, 80), (1, 0, 3, 2))]
    for shape, axes in cases:
        base = to_dtype(rng.standard_normal(shape), dtype)
        got = ag.Tensor.from_array(base).permuted_axes(axes).to_standard_layout().into_array()
        assert np.array_equal(got, orc.to_standard_layout(base.transpose(axes))), (shape, axes)
    # a view at an odd element offset with an odd row stride: the element-wise tiles
    big = to_dtype(rng.standard_normal((3, 131, 77)), dtype)
    t = ag.Tensor.from_array(big)
    view = ag.Tensor(t.buffer, (3, 64, 129), (131 * 77, 1, 77), 1 * 77 + 5, dtype)  # big[:, 1:130, 5:69] transposed
    assert np.array_equal(view.to_standard_layout().into_array(), np.ascontiguousarray(big[:, 1:130, 5:69].transpose(0, 2, 1)))
    # the benchmark's activation, NHWC -> NCHW and back
    act = to_dtype(rng.standard_normal((256, 56, 56, 128), dtype=np.float32), dtype)
    nchw = ag.Tensor.from_array(act).permuted_axes((0, 3, 1, 2)).to_standard_layout()
    assert np.array_equal(nchw.into_array(), orc.to_standard_layout(act.transpose(0, 3, 1, 2)))
    back = nchw.permuted_axes((0, 2, 3, 1)).to_standard_layout().into_array()
    assert np.array_equal(back, act)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_scaled_add_sgd_sum_axis0_bit_exact(ag, dtype):
    rng = np.random.default_rng(42)
    for n in (1, 255, 46920, 300001):
        y, x, v = (to_dtype(rng.standard_normal(n), dtype) for _ in range(3))
        ty = ag.Tensor.from_array(y)
        ty.scaled_add(-0.01, ag.Tensor.from_array(x))
        assert np.array_equal(ty.into_array(), orc.scaled_add(y, -0.01, x))
        tw, tv = ag.Tensor.from_array(y), ag.Tensor.from_array(v)
        ag.SGD(momentum=0.9).update(0.01, tw, ag.Tensor.from_array(x), tv)
        w2, v2 = orc.sgd_momentum(y, x, 0.01, 0.9, v)
        assert np.array_equal(tw.into_array(), w2) and np.array_equal(tv.into_array(), v2)
    for rows, cols in [(100, 10), (1, 7), (1000, 300), (257, 1)]:
        a = to_dtype(rng.standard_normal((rows, cols)) * 4, dtype)
        assert np.array_equal(ag.Tensor.from_array(a).sum_axis0().into_array(), orc.sum_axis0(a))
    a = to_dtype(np.array([[256.0, 1.0]] + [[1.0, 1.0]] * 64), dtype)
    assert np.array_equal(ag.Tensor.from_array(a).sum_axis0().into_array(), orc.sum_axis0(a))


def _view_of(ag, t, a, base):
    """The device Tensor that shows the same elements of `t` (uploaded from `base`) as the numpy view `a` of `base`."""
    es = base.itemsize
    off = (a.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // es
    return ag.Tensor(t.buffer, a.shape, tuple(st // es for st in a.strides), off, t.dtype)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_scaled_add_on_strided_and_broadcast_views(ag, dtype):
    """`scaled_add` / `add_assign` on views (src/tensor/ops.rs:192-204, :245-255, :257-318): bit-exact against the
    oracle, elements outside the destination view untouched; the 16-byte form (aligned, contiguous innermost axis) and
    the element-wise one, negative strides, offsets, stride-0 sources, the Dense bias at full size."""
    rng = np.random.default_rng(45)
    base = to_dtype(rng.standard_normal((6, 10, 12, 16)), dtype)

    def run(yview, x, alpha):
        want = base.copy()
        orc.scaled_add_strided(yview(want), alpha, x)
        ty = ag.Tensor.from_array(base)
        tx = ag.Tensor.from_array(x)
        _view_of(ag, ty, yview(base), base).scaled_add(alpha, tx)
        assert np.array_equal(ty.into_array(), want)

    mk = lambda *shape: to_dtype(rng.standard_normal(shape) * 3, dtype)
    run(lambda a: a, mk(16), 1.0)                                   # bias over the trailing axis, 16-byte groups
    run(lambda a: a, mk(6, 1, 12, 1), -0.01)                        # stride-0 innermost source
    run(lambda a: a[:, ::2, 1:9, :], mk(5, 8, 16), 0.3)             # sliced destination, still vectorisable
    run(lambda a: a[:, :, :, 3:11], mk(12, 8), 0.3)                 # unaligned innermost window
    run(lambda a: a.transpose(0, 3, 1, 2), mk(16, 10, 12), 2.0)     # permuted destination (NHWC buffer seen as NCHW)
    run(lambda a: a[::-1, :, ::-1, ::-2], mk(1,), 0.5)              # negative strides, scalar source
    run(lambda a: a[2, 3], mk(12, 16), -1.0)                        # 2-D window at an offset
    # source given as a strided view itself (a transposed matrix), destination contiguous
    y = to_dtype(rng.standard_normal((300, 70)), dtype)
    x = to_dtype(rng.standard_normal((70, 300)), dtype)
    ty, tx = ag.Tensor.from_array(y), ag.Tensor.from_array(x)
    ty.scaled_add(0.25, tx.t())
    want = y.copy()
    orc.scaled_add_strided(want, 0.25, x.T)
    assert np.array_equal(ty.into_array(), want)
    # y += y (aliasing element for element)
    ty = ag.Tensor.from_array(y)
    tyt = ty.t()
    tyt.add_assign(tyt)
    want = y.copy()
    orc.scaled_add_strided(want.T, 1.0, want.T.copy())
    assert np.array_equal(ty.into_array(), want)
    # shapes that cannot broadcast, a broadcast destination and a type mismatch are refused before any launch
    with pytest.raises(ag.AghError, match="Broadcast not possible"):
        ty.scaled_add(1.0, ag.Tensor.from_array(mk(7)))
    with pytest.raises(ag.AghError, match="destination cannot be a broadcast view"):
        ag.Tensor.from_array(mk(70)).broadcast((300, 70)).scaled_add(1.0, ty)
    with pytest.raises(ag.AghError):
        ty.scaled_add(1.0, ag.Tensor.from_array(to_dtype(rng.standard_normal((300, 70)), "f32" if dtype == "bf16" else "bf16")))
    # the Dense-shaped bias add at full size, [16384, 4096] += [4096]
    big = to_dtype(rng.standard_normal((16384, 4096), dtype=np.float32), dtype)
    bias = mk(4096)
    tb = ag.Tensor.from_array(big)
    tb.add_assign(ag.Tensor.from_array(bias))
    assert np.array_equal(tb.into_array(), orc.bias_add_rows(big, bias))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_dense_unfused_equals_fused_epilogue(ag, dtype):
    """`Dense::forward` as the reference issues it (layer.rs:1137-1140: dot, `add_assign(&bias)`, then the Relu layer)
    against the one-launch epilogue: the same bits."""
    rng = np.random.default_rng(46)
    for m, k, n in [(100, 84, 10), (1000, 256, 128), (257, 1000, 333), (2048, 512, 1024)]:
        x = ag.Tensor.from_array(to_dtype(rng.standard_normal((m, k)), dtype))
        layer = ag.Dense(ag.Tensor.from_array(to_dtype(rng.standard_normal((k, n)) * 0.1, dtype)),
                         ag.Tensor.from_array(to_dtype(rng.standard_normal(n), dtype)))
        for relu in (False, True):
            a, b = layer.forward(x, relu=relu).into_array(), layer.forward(x, relu=relu, fused=False).into_array()
            assert np.array_equal(a, b), (m, k, n, relu)
        plain = x.dot(layer.weight).into_array()
        assert np.array_equal(layer.forward(x, fused=False).into_array(), orc.bias_add_rows(plain, layer.bias.into_array()))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_accuracy(ag, dtype):
    """`Accuracy` (src/learn/criterion.rs:22-118): the reference test's generator (tests/integration_tests.rs:767-793),
    ties / NaNs / out-of-range targets, and random data with many ties at sizes that take one and several workgroups."""
    for bs, classes in [(1, 8), (31, 16), (1000, 100)]:
        flat = np.resize(np.arange(classes), bs * classes + classes // 2 + 1)[classes // 2 + 1:][: bs * classes]
        x = to_dtype(flat.reshape(bs, classes), dtype)
        t = (np.arange(bs) % classes).astype(np.uint8)
        assert ag.Tensor.from_array(x).accuracy(labels(ag, t)) == orc.accuracy(x, t)
    x = to_dtype(np.array([[1, 3, 2], [3, 3, 1], [np.nan, 1, 0], [0, np.nan, 5], [2, 1, 0], [-0.0, 0.0, -1]]), dtype)
    t = np.array([1, 0, 0, 2, 7, 0], dtype=np.uint8)
    assert ag.Tensor.from_array(x).accuracy(labels(ag, t)) == orc.accuracy(x, t) == 1
    rng = np.random.default_rng(47)
    for bs, classes in [(5000, 6), (300000, 10), (70000, 256)]:
        x = to_dtype(rng.integers(0, 3 if classes < 100 else 4000, (bs, classes)), dtype)
        t = rng.integers(0, classes, bs).astype(np.uint8)
        want = orc.accuracy(x, t)
        assert 0 < want < bs
        assert ag.Tensor.from_array(x).accuracy(labels(ag, t)) == want
    # the count may go straight to pinned host memory
    hp = C.c_void_p()
    ag._ffi.check(ag.lib.agh_host_alloc(C.byref(hp), 4))
    tx = ag.Tensor.from_array(x)
    ag._ffi.check(getattr(ag.lib, f"agh_accuracy_{dtype}")(tx._data_ptr(), labels(ag, t).ptr, bs, classes, hp))
    ag._ffi.check(ag.lib.agh_sync())
    assert C.cast(hp, C.POINTER(C.c_uint32))[0] == want
    ag._ffi.check(ag.lib.agh_host_free(hp))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_cross_entropy(ag, dtype):
    rng = np.random.default_rng(43)
    for bs, classes in [(100, 10), (7, 3), (1000, 10), (513, 256)]:
        x = to_dtype(rng.standard_normal((bs, classes)) * 3, dtype)
        t = rng.integers(0, classes, bs).astype(np.uint8)
        tx, tt = ag.Tensor.from_array(x), labels(ag, t)
        want = orc.cross_entropy_loss(x, t)
        got = tx.cross_entropy_loss(tt)
        assert abs(got - want) <= 2e-6 * bs + 1e-6 * abs(want), (got, want)  # expf / logf differ by an ulp or two
        g = tx.cross_entropy_loss_backward(tt).into_array()
        wg = orc.cross_entropy_backward(x, t)
        if dtype == "f32":
            assert np.all(np.abs(g - wg) <= 4e-6 * np.abs(wg) + 1e-9)
        else:
            gf, wf = as_f32(g).astype(np.float64), as_f32(wg).astype(np.float64)
            assert np.all(np.abs(gf - wf) <= 2.0**-7 * np.abs(wf))  # at most one bf16 step apart
            assert np.mean(g != wg) < 0.01
    x = to_dtype(np.array([[1000.0, 999.0, -1000.0]]), dtype)
    tt = labels(ag, np.array([1], dtype=np.uint8))
    assert abs(ag.Tensor.from_array(x).cross_entropy_loss(tt) - orc.cross_entropy_loss(x, np.array([1], dtype=np.uint8))) < 1e-5


def he(rng, shape, fan_in):
    a = np.sqrt(2.0 / fan_in)
    return rng.uniform(-a, a, shape).astype(np.float32)


def lenet_params(rng):
    return [he(rng, (6, 1, 5, 5), 25), he(rng, (16, 6, 5, 5), 150), he(rng, (256, 128), 256), he(rng, (128, 84), 128),
            he(rng, (84, 10), 84), he(rng, (10,), 84)]


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("bs", [100, 3])
def test_lenet5_forward_train_saves_every_activation(ag, dtype, bs):
    """agh_lenet5_forward_train_<T>: the forward pass of a training step in one launch.  Every saved activation must be
    what the reference's layer produces from the PREVIOUS saved activation (layer.rs:950-1005, :1134-1143, :1193-1216,
    :1253-1267): convolutions and dense layers within the GEMM tolerances of the oracle's result on that very
    input (they sum in f32 in another order), relu and pooling bit for bit."""
    rng = np.random.default_rng(47)
    params = [to_dtype(p, dtype) for p in lenet_params(rng)]
    w1, w2, wd1, wd2, wd3, b3 = params
    x = to_dtype(rng.uniform(0, 1, (bs, 1, 28, 28)), dtype)
    shapes = [(bs, 6, 24, 24), (bs, 6, 12, 12), (bs, 16, 8, 8), (bs, 16, 4, 4), (bs, 128), (bs, 128), (bs, 84), (bs, 84), (bs, 10)]
    outs = [ag.Tensor.zeros(sh, dtype) for sh in shapes]
    tp = [ag.Tensor.from_array(p) for p in params]
    tx = ag.Tensor.from_array(x)
    ag._ffi.check(getattr(ag.lib, f"agh_lenet5_forward_train_{dtype}")(tx._ptr(), *[t._ptr() for t in tp], *[o._ptr() for o in outs], bs))
    c1, p1, c2, p2, d1, a1, d2, a2, logits = [o.into_array() for o in outs]

    def close(got, want64, scale64, k):
        g = as_f32(got).astype(np.float64)
        if dtype == "f32":
            assert np.all(np.abs(g - want64) <= 1e-5 * np.sqrt(k) * scale64 + 1e-30)
        else:
            ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want64), 2.0**-126))) - 7)
            assert np.all(np.abs(g - want64) <= ulp + 1e-2 * np.abs(want64) + 8 * np.sqrt(k) * 2.0**-24 * scale64)

    f = as_f32
    close(c1, orc.conv2_naive_f64(f(x), f(w1)), orc.conv2_naive_f64(np.abs(f(x)), np.abs(f(w1))), 25)
    assert np.array_equal(p1, orc.max_pool2(orc.relu(c1), (2, 2)))
    close(c2, orc.conv2_naive_f64(f(p1), f(w2)), orc.conv2_naive_f64(np.abs(f(p1)), np.abs(f(w2))), 150)
    assert np.array_equal(p2, orc.max_pool2(orc.relu(c2), (2, 2)))
    flat = f(p2).reshape(bs, 256).astype(np.float64)
    close(d1, flat @ f(wd1).astype(np.float64), np.abs(flat) @ np.abs(f(wd1)).astype(np.float64), 256)
    assert np.array_equal(a1, orc.relu(d1))
    a1f = f(a1).astype(np.float64)
    close(d2, a1f @ f(wd2).astype(np.float64), np.abs(a1f) @ np.abs(f(wd2)).astype(np.float64), 128)
    assert np.array_equal(a2, orc.relu(d2))
    a2f = f(a2).astype(np.float64)
    # dense3: T(dot) then T(. + bias): one more rounding step than a plain product
    want = a2f @ f(wd3).astype(np.float64) + f(b3).astype(np.float64)
    scale = np.abs(a2f) @ np.abs(f(wd3)).astype(np.float64) + np.abs(f(b3)).astype(np.float64)
    g = f(logits).astype(np.float64)
    if dtype == "f32":
        assert np.all(np.abs(g - want) <= 1e-5 * np.sqrt(84) * scale)
    else:
        ulp = 2.0 ** (np.floor(np.log2(np.maximum(scale, 2.0**-126))) - 7)
        assert np.all(np.abs(g - want) <= 2 * ulp + 1e-2 * np.abs(want))
    # the logits are those of the inference launch, bit for bit (same kernel body)
    inf = ag.Tensor.zeros((bs, 10), dtype)
    ag._ffi.check(getattr(ag.lib, f"agh_lenet5_forward_{dtype}")(tx._ptr(), *[t._ptr() for t in tp], inf._ptr(), bs))
    assert np.array_equal(inf.into_array(), logits)
    with pytest.raises(ag.AghError):  # a missing buffer is an error, never a launch
        ag._ffi.check(getattr(ag.lib, f"agh_lenet5_forward_train_{dtype}")(tx._ptr(), *[t._ptr() for t in tp],
                                                                         *[o._ptr() for o in outs[:3]], None, *[o._ptr() for o in outs[4:]], bs))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_lenet5_backward_one_launch_against_the_separate_launches(ag, dtype):
    """agh_lenet5_backward_<T> against the nine launches it replaces, on the same activations: the cross-entropy
    gradient bit for bit, the rest up to the summation order of the dense dot products (every rounding point and the
    order of the T-typed col2im sums are the same)."""
    rng = np.random.default_rng(46)
    params = [to_dtype(p, dtype) for p in lenet_params(rng)]
    bs = 100
    x = to_dtype(rng.uniform(0, 1, (bs, 1, 28, 28)), dtype)
    t = rng.integers(0, 10, bs).astype(np.uint8)
    tx, tt = ag.Tensor.from_array(x), labels(ag, t)
    got, want = {}, {}
    for fused, out in ((True, got), (False, want)):
        tr = ag.LeNet5Trainer(ag.LeNet5.from_arrays(*params), bs, optimizer=ag.SGD(None), overlap=False,
                              fused_forward=True, fused_backward=fused)
        tr.step(tx, tt)
        ag._ffi.check(ag.lib.agh_sync())
        for name in ("g_logits", "g_d2", "g_d1", "gm2", "gm1"):
            out[name] = as_f32(getattr(tr, name).into_array()).astype(np.float64)
        out["loss"] = tr.loss()
        for name, g in zip(("dw1", "dw2", "dwd1", "dwd2", "dwd3", "db3"), tr.grads):
            out[name] = as_f32(g.into_array()).astype(np.float64)
    assert np.array_equal(got["g_logits"], want["g_logits"])
    # same rows added in the same order: the bias gradient and the loss of agh_lenet5_dense_weight_grads_<T> are those of
    # agh_sum_axis0_<T> / agh_cross_entropy_loss_<T> bit for bit; dwd3 multiplies identical operands in another order
    assert np.array_equal(got["db3"], want["db3"]) and got["loss"] == want["loss"]
    assert np.abs(got["dwd3"] - want["dwd3"]).max() <= (1e-5 if dtype == "f32" else 2.0**-7) * np.abs(want["dwd3"]).max()
    for name in ("dw1", "dw2", "dwd1", "dwd2"):
        sc = np.abs(want[name]).max()
        assert np.abs(got[name] - want[name]).max() <= (1e-4 if dtype == "f32" else 2.0**-5) * sc, name
    for name in ("g_d2", "g_d1", "gm2", "gm1"):
        g, w = got[name], want[name]
        scale = np.abs(w).max()
        assert scale > 0
        assert np.array_equal(g == 0, w == 0) or np.mean((g == 0) != (w == 0)) < 1e-3, name  # same relu / pooling decisions
        if dtype == "f32":
            assert np.abs(g - w).max() <= 1e-5 * scale, name
        else:
            assert np.abs(g - w).max() <= 2.0**-6 * scale and np.abs(g - w).mean() <= 2.0**-11 * scale, name


@pytest.mark.parametrize("fused_backward", [True, False])
@pytest.mark.parametrize("fused_forward", [True, False])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("momentum", [None, 0.01])
def test_lenet5_train_step(ag, dtype, momentum, fused_forward, fused_backward):
    rng = np.random.default_rng(44)
    params = [to_dtype(p, dtype) for p in lenet_params(rng)]
    bs = 100
    x = to_dtype(rng.uniform(0, 1, (bs, 1, 28, 28)), dtype)
    t = rng.integers(0, 10, bs).astype(np.uint8)
    inter = {}
    want_loss, want_params, want_grads, want_v = orc.lenet5_train_step(x, t, params, lr=0.01, momentum=momentum, intermediates=inter)

    model = ag.LeNet5.from_arrays(*params)
    trainer = ag.LeNet5Trainer(model, bs, learning_rate=0.01, optimizer=ag.SGD(momentum), fused_forward=fused_forward,
                               fused_backward=fused_backward)
    tx, tt = ag.Tensor.from_array(x), labels(ag, t)
    trainer.step(tx, tt)
    ag._ffi.check(ag.lib.agh_sync())
    assert abs(trainer.loss() - want_loss) <= (1e-5 if dtype == "f32" else 1e-2) * abs(want_loss)
    for name, g, w in zip(("dw1", "dw2", "dwd1", "dwd2", "dwd3", "db3"), trainer.grads, want_grads):
        gf, wf = as_f32(g.into_array()).astype(np.float64), as_f32(w).astype(np.float64)
        scale = np.abs(wf).max()
        if dtype == "f32":
            # f32 sums in another order (k up to 57600 for dw1): 1e-5 * sqrt(k) of the scale
            assert np.abs(gf - wf).max() <= 3e-3 * scale, name
        else:
            # bf16: every GEMM may differ from the oracle's by one rounding, and a flipped relu / pool
            # decision moves single entries; the bulk has to agree
            assert np.abs(gf - wf).max() <= 0.1 * scale, name
            assert np.abs(gf - wf).mean() <= 0.01 * scale, name
    # The masked gradients of the backward chain: a wrong relu or pooling mask moves whole cells between zero and
    # non-zero, which the tolerances above would not see.  The zero pattern has to be the oracle's except where the
    # last bit of a forward dot product decides a sign or a maximum (measured: under 0.1 % of the cells), and on the
    # cells both call non-zero the values agree to a few bf16 steps of the tensor's scale.
    for name in ("g_logits", "g_d2", "g_d1", "gm2", "gm1"):
        g = as_f32(getattr(trainer, name).into_array()).astype(np.float64)
        w = as_f32(inter[name]).astype(np.float64).reshape(g.shape)
        flips = np.mean((g == 0) != (w == 0))
        assert flips <= 2e-3, (name, flips)
        assert 0.02 < np.mean(w == 0) < 0.98 or name == "g_logits", name  # the masks are really there
        both = (g != 0) & (w != 0)
        scale = np.abs(w).max()
        err = np.abs(g - w)[both]
        assert err.max() <= (1e-4 if dtype == "f32" else 2.0**-5) * scale, name
        assert err.mean() <= (1e-6 if dtype == "f32" else 2.0**-10) * scale, name
    for name, p, w, old in zip(("w1", "w2", "wd1", "wd2", "wd3", "b3"), trainer.params, want_params, params):
        pf, wf, of = (as_f32(a).astype(np.float64) for a in (p.into_array(), w, old))
        step = np.abs(wf - of).max()
        assert np.abs(pf - wf).max() <= (3e-3 if dtype == "f32" else 0.1) * step + (0 if dtype == "f32" else 2.0**-8 * np.abs(wf).max()), name
    # the update itself is exact: applying the oracle's update to the GPU's own gradients gives the GPU's parameters
    for p, old, g, v in zip(trainer.params, params, trainer.grads, trainer.velocities):
        ga = g.into_array()
        if momentum is None:
            assert np.array_equal(p.into_array(), orc.scaled_add(old, -0.01, ga))
        else:
            w2, v2 = orc.sgd_momentum(old, ga, 0.01, momentum, np.zeros_like(old))
            assert np.array_equal(p.into_array(), w2) and np.array_equal(v.into_array(), v2)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_lenet5_train_graph_replay_equals_eager(ag, dtype):
    rng = np.random.default_rng(45)
    params = [to_dtype(p, dtype) for p in lenet_params(rng)]
    bs = 100
    x = to_dtype(rng.uniform(0, 1, (bs, 1, 28, 28)), dtype)
    t = rng.integers(0, 10, bs).astype(np.uint8)
    tx, tt = ag.Tensor.from_array(x), labels(ag, t)
    # the eager steps on one stream, the graph with the weight gradients on the second stream
    eager = ag.LeNet5Trainer(ag.LeNet5.from_arrays(*params), bs, optimizer=ag.SGD(0.01), overlap=False)
    graph = ag.LeNet5Trainer(ag.LeNet5.from_arrays(*params), bs, optimizer=ag.SGD(0.01))
    graph.capture(tx, tt)  # two steps: one eager, one while recording... recording does not execute
    losses = []
    for i in range(3):
        eager.step(tx, tt)
        ag._ffi.check(ag.lib.agh_sync())
        losses.append(eager.loss())
    # capture() ran ONE real step (work recorded during capture is not executed); two replays follow
    for i in range(2):
        graph.replay()
        ag._ffi.check(ag.lib.agh_sync())
        assert graph.loss() == losses[i + 1], i
    for a, b in zip(eager.params, graph.params):
        assert np.array_equal(a.into_array(), b.into_array())
    assert losses[2] < losses[0]  # three steps on the same batch lower its loss


def test_branch_join_matches_one_stream(ag):
    """Two products of one left operand (a layer's weight and input gradients, autograd.rs:607-627), the
    first on the second stream: same bits as in order on one stream, eagerly and in a replayed graph."""
    rng = np.random.default_rng(46)
    g = ag.Tensor.from_array(rng.standard_normal((300, 84)).astype(np.float32))
    a = ag.Tensor.from_array(rng.standard_normal((300, 120)).astype(np.float32))
    w = ag.Tensor.from_array(rng.standard_normal((120, 84)).astype(np.float32))
    dw0, da0 = ag.Tensor.zeros((120, 84), "f32"), ag.Tensor.zeros((300, 120), "f32")
    ag.gemm(1.0, a.t(), g, 0.0, dw0)
    ag.gemm(1.0, g, w.t(), 0.0, da0)
    want_dw, want_da = dw0.into_array(), da0.into_array()

    def forked(dw, da):
        with ag.branch():
            ag.gemm(1.0, a.t(), g, 0.0, dw)
        ag.gemm(1.0, g, w.t(), 0.0, da)
        ag.join()

    dw1, da1 = ag.Tensor.zeros((120, 84), "f32"), ag.Tensor.zeros((300, 120), "f32")
    forked(dw1, da1)
    assert np.array_equal(dw1.into_array(), want_dw) and np.array_equal(da1.into_array(), want_da)

    # misuse is an error, and leaves the library usable
    with pytest.raises(ag.AghError):
        ag._ffi.check(ag.lib.agh_branch_end())
    ag._ffi.check(ag.lib.agh_branch_begin())
    with pytest.raises(ag.AghError):
        ag._ffi.check(ag.lib.agh_branch_begin())
    with pytest.raises(ag.AghError):
        ag._ffi.check(ag.lib.agh_branch_join())
    ag._ffi.check(ag.lib.agh_branch_end())
    ag.join()

    dw2, da2 = ag.Tensor.zeros((120, 84), "f32"), ag.Tensor.zeros((300, 120), "f32")
    ag._ffi.check(ag.lib.agh_sync())
    ag._ffi.check(ag.lib.agh_graph_begin())
    try:
        forked(dw2, da2)
    finally:
        graph = C.c_void_p()
        ag._ffi.check(ag.lib.agh_graph_end(C.byref(graph)))
    try:
        zero = np.zeros((120, 84), np.float32)
        for _ in range(3):
            ag._ffi.check(ag.lib.agh_memcpy_h2d(dw2._ptr(), zero.ctypes.data, zero.nbytes))
            ag._ffi.check(ag.lib.agh_graph_launch(graph))
            assert np.array_equal(dw2.into_array(), want_dw) and np.array_equal(da2.into_array(), want_da)
    finally:
        ag._ffi.check(ag.lib.agh_graph_destroy(graph))
