"""ctypes front end of the CPU oracle (``oracle.c``).

Test infrastructure only: tests/, the smoke check and the bench's cpu_baseline leg
load this; the product package never does.  All arrays are numpy; bf16 tensors are
``uint16`` arrays holding the raw bit patterns.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def _load():
    if not os.path.exists(_SO):
        build()
    return C.CDLL(_SO)


_lib = _load()
_i64 = C.c_int64
_p = C.c_void_p


def _ptr(a):
    return a.ctypes.data_as(_p)


def _sig(name, args, res=None):
    f = getattr(_lib, name)
    f.argtypes = args
    f.restype = res
    return f


_sig("orc_f32_to_bf16_n", [_p, _p, _i64])
_sig("orc_bf16_to_f32_n", [_p, _p, _i64])
_sig("orc_conv_out", [_i64] * 5, _i64)
_sig("orc_col2im_out", [_i64] * 5, _i64)
_sig("orc_pool_out", [_i64] * 3, _i64)
for _n in ("orc_im2col_conv2_b32", "orc_im2col_conv2_b16", "orc_col2im_conv2_f32", "orc_col2im_conv2_bf16"):
    _sig(_n, [_p, _p] + [_i64] * 12)
for _n in ("orc_max_pool2_f32", "orc_max_pool2_bf16", "orc_max_pool2_backward_f32", "orc_max_pool2_backward_bf16"):
    _sig(_n, [_p, _p] + [_i64] * 7)
_sig("orc_relu_f32", [_p, _p, _i64])
_sig("orc_relu_bf16", [_p, _p, _i64])
_sig("orc_relu_backward_f32", [_p, _p, _p, _i64])
_sig("orc_relu_backward_bf16", [_p, _p, _p, _i64])
_sig("orc_bias_add_rows_f32", [_p, _p, _i64, _i64])
_sig("orc_bias_add_rows_bf16", [_p, _p, _i64, _i64])
_g = [_i64, _i64, _i64]
_v = [_p, _i64, _i64, _i64]
_sig("orc_gemm_f32_f64acc", _g + [C.c_double] + _v + _v + [C.c_double, _p, _p, _i64, _i64, _i64])
_sig("orc_gemm_bf16_f64acc", _g + [C.c_double] + _v + _v + [C.c_double, _p, _p, _i64, _i64, _i64])
_sig("orc_gemm_bf16_f32acc", _g + [C.c_float] + _v + _v + [C.c_float] + _v)
_sig("orc_gemm_bf16_hostfold", _g + _v + _v + [_p])
_sig("orc_gemm_f32_host", _g + [C.c_float] + _v + _v + [C.c_float] + _v + [C.c_int])
_sig("orc_conv2_naive_f64", [_p, _p, _p] + [_i64] * 13)
_sig("orc_lenet5_forward_f32", [_p, _i64, _p, _p, _p, _p, _p, _p, _p, C.c_int])
_sig("orc_lenet5_forward_f32_alg", [_p, _i64, _p, _p, _p, _p, _p, _p, _p, C.c_int, C.c_int])
_sig("orc_conv2_direct_f32", [_p, _p, _p] + [_i64] * 7)
_sig("orc_conv2_direct_packed_f32", [_p, _p, _p] + [_i64] * 7 + [C.c_int])
_sig("orc_max_threads", [], C.c_int)
_sig("orc_assign4", [_p, _i64, _p, _p, _i64, _p, _p, _i64])
_sig("orc_scaled_add_f32", [_p, C.c_float, _p, _i64])
_sig("orc_scaled_add_bf16", [_p, C.c_float, _p, _i64])
_sig("orc_scaled_add_strided_f32", [_p, _i64, _p, C.c_float, _p, _i64, _p, _p])
_sig("orc_scaled_add_strided_bf16", [_p, _i64, _p, C.c_float, _p, _i64, _p, _p])
_sig("orc_accuracy_f32", [_p, _p, _i64, _i64], _i64)
_sig("orc_accuracy_bf16", [_p, _p, _i64, _i64], _i64)
_sig("orc_sgd_momentum_f32", [_p, _p, C.c_float, C.c_float, _p, _i64])
_sig("orc_sgd_momentum_bf16", [_p, _p, C.c_float, C.c_float, _p, _i64])
_sig("orc_sum_axis0_f32", [_p, _p, _i64, _i64])
_sig("orc_sum_axis0_bf16", [_p, _p, _i64, _i64])
_sig("orc_cross_entropy_loss_f32", [_p, _p, _i64, _i64], C.c_float)
_sig("orc_cross_entropy_loss_bf16", [_p, _p, _i64, _i64], C.c_float)
_sig("orc_cross_entropy_backward_f32", [_p, _p, C.c_float, _p, _i64, _i64])
_sig("orc_cross_entropy_backward_bf16", [_p, _p, C.c_float, _p, _i64, _i64])


def max_threads():
    return int(_lib.orc_max_threads())


# ---------------------------------------------------------------- bf16 ----
def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.uint16)
    _lib.orc_f32_to_bf16_n(_ptr(x), _ptr(y), x.size)
    return y


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty(x.shape, dtype=np.float32)
    _lib.orc_bf16_to_f32_n(_ptr(x), _ptr(y), x.size)
    return y


# -------------------------------------------------------------- shapes ----
def conv_out(i, f, p=0, s=1, d=1):
    return int(_lib.orc_conv_out(i, f, p, s, d))


def col2im_out(i, f, p=0, s=1, d=1):
    return int(_lib.orc_col2im_out(i, f, p, s, d))


def pool_out(i, x, s):
    return int(_lib.orc_pool_out(i, x, s))


def _is_bf16(a):
    return a.dtype == np.uint16


# -------------------------------------------------------------- im2col ----
def im2col_conv2(x, filter, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
    x = np.ascontiguousarray(x)
    bs, c, ih, iw = x.shape
    (fh, fw), (ph, pw), (sh, sw), (dh, dw) = filter, padding, stride, dilation
    oh, ow = conv_out(ih, fh, ph, sh, dh), conv_out(iw, fw, pw, sw, dw)
    y = np.empty((bs * oh * ow, c * fh * fw), dtype=x.dtype)
    fn = _lib.orc_im2col_conv2_b16 if x.dtype.itemsize == 2 else _lib.orc_im2col_conv2_b32
    assert x.dtype.itemsize in (2, 4)
    fn(_ptr(x), _ptr(y), bs, c, ih, iw, fh, fw, ph, pw, sh, sw, dh, dw)
    return y


def col2im_conv2(x, shape, filter, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
    """x: [bs*ih*iw, c*fh*fw] with shape=(ih, iw) the patch grid."""
    x = np.ascontiguousarray(x)
    (ih, iw), (fh, fw), (ph, pw), (sh, sw), (dh, dw) = shape, filter, padding, stride, dilation
    rows, cols = x.shape
    bs, c = rows // (ih * iw), cols // (fh * fw)
    oh, ow = col2im_out(ih, fh, ph, sh, dh), col2im_out(iw, fw, pw, sw, dw)
    y = np.empty((bs, c, oh, ow), dtype=x.dtype)
    fn = _lib.orc_col2im_conv2_bf16 if _is_bf16(x) else _lib.orc_col2im_conv2_f32
    assert x.dtype in (np.uint16, np.float32)
    fn(_ptr(x), _ptr(y), bs, c, ih, iw, fh, fw, ph, pw, sh, sw, dh, dw)
    return y


# ---------------------------------------------------------------- pool ----
def max_pool2(x, size, strides=None):
    strides = strides or size
    x = np.ascontiguousarray(x)
    bs, c, ih, iw = x.shape
    oh, ow = pool_out(ih, size[0], strides[0]), pool_out(iw, size[1], strides[1])
    y = np.empty((bs, c, oh, ow), dtype=x.dtype)
    fn = _lib.orc_max_pool2_bf16 if _is_bf16(x) else _lib.orc_max_pool2_f32
    fn(_ptr(x), _ptr(y), bs * c, ih, iw, size[0], size[1], strides[0], strides[1])
    return y


def max_pool2_backward(x, dy, size, strides=None):
    """Returns dx; `x` is the forward input (copied, as the layer's edge does)."""
    strides = strides or size
    dx = np.array(x, order="C", copy=True)
    dy = np.ascontiguousarray(dy)
    bs, c, ih, iw = dx.shape
    fn = _lib.orc_max_pool2_backward_bf16 if _is_bf16(dx) else _lib.orc_max_pool2_backward_f32
    fn(_ptr(dx), _ptr(dy), bs * c, ih, iw, size[0], size[1], strides[0], strides[1])
    return dx


# ---------------------------------------------------------- relu / bias ----
def relu(x):
    x = np.ascontiguousarray(x)
    y = np.empty_like(x)
    (_lib.orc_relu_bf16 if _is_bf16(x) else _lib.orc_relu_f32)(_ptr(x), _ptr(y), x.size)
    return y


def relu_backward(x, dy):
    x, dy = np.ascontiguousarray(x), np.ascontiguousarray(dy)
    dx = np.empty_like(x)
    (_lib.orc_relu_backward_bf16 if _is_bf16(x) else _lib.orc_relu_backward_f32)(_ptr(x), _ptr(dy), _ptr(dx), x.size)
    return dx


def bias_add_rows(y, bias):
    y = np.array(y, order="C", copy=True)
    bias = np.ascontiguousarray(bias)
    m, n = y.shape
    (_lib.orc_bias_add_rows_bf16 if _is_bf16(y) else _lib.orc_bias_add_rows_f32)(_ptr(y), _ptr(bias), m, n)
    return y


# ---------------------------------------------------------------- gemm ----
def _view(a):
    """(base array, element offset, row stride, col stride) of a 2-D numpy view, in elements."""
    base = a
    while base.base is not None and isinstance(base.base, np.ndarray):
        base = base.base
    es = a.dtype.itemsize
    off = (a.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // es
    return base, off, a.strides[0] // es, a.strides[1] // es


def gemm_f64acc(a, b, alpha=1.0, beta=0.0, c=None):
    """Checker: f64-accumulated alpha*a@b + beta*c for f32 or bf16(uint16) views; returns f64 [m,n]."""
    m, k = a.shape
    k2, n = b.shape
    assert k == k2
    ab, oa, rsa, csa = _view(a)
    bb, ob, rsb, csb = _view(b)
    out = np.empty((m, n), dtype=np.float64)
    if c is None:
        cb, oc, rsc, csc, cp = None, 0, 0, 0, None
    else:
        cb, oc, rsc, csc = _view(c)
        cp = _ptr(cb)
    fn = _lib.orc_gemm_bf16_f64acc if _is_bf16(a) else _lib.orc_gemm_f32_f64acc
    fn(m, k, n, alpha, _ptr(ab), oa, rsa, csa, _ptr(bb), ob, rsb, csb, beta if c is not None else 0.0, cp,
       _ptr(out), oc, rsc, csc)
    return out


def gemm_bf16_f32acc(a, b, alpha=1.0, beta=0.0, c=None):
    """The reference device kernel's numerics: f32 accumulate, single RNE; returns uint16 [m,n]."""
    m, k = a.shape
    _, n = b.shape
    ab, oa, rsa, csa = _view(a)
    bb, ob, rsb, csb = _view(b)
    out = np.zeros((m, n), dtype=np.uint16) if c is None else np.array(c, order="C", copy=True)
    _lib.orc_gemm_bf16_f32acc(m, k, n, alpha, _ptr(ab), oa, rsa, csa, _ptr(bb), ob, rsb, csb,
                              beta if c is not None else 0.0, _ptr(out), 0, n, 1)
    return out


def gemm_bf16_hostfold(a, b):
    m, k = a.shape
    _, n = b.shape
    ab, oa, rsa, csa = _view(a)
    bb, ob, rsb, csb = _view(b)
    out = np.empty((m, n), dtype=np.uint16)
    _lib.orc_gemm_bf16_hostfold(m, k, n, _ptr(ab), oa, rsa, csa, _ptr(bb), ob, rsb, csb, _ptr(out))
    return out


def gemm_f32_host(a, b, alpha=1.0, beta=0.0, c=None, threads=4):
    m, k = a.shape
    _, n = b.shape
    ab, oa, rsa, csa = _view(a)
    bb, ob, rsb, csb = _view(b)
    out = np.zeros((m, n), dtype=np.float32) if c is None else np.array(c, order="C", copy=True)
    _lib.orc_gemm_f32_host(m, k, n, alpha, _ptr(ab), oa, rsa, csa, _ptr(bb), ob, rsb, csb,
                           beta if c is not None else 0.0, _ptr(out), 0, n, 1, threads)
    return out


# ---------------------------------------------------------------- conv ----
def conv2_naive_f64(x, w, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    bs, ic, ih, iw = x.shape
    oc, ic2, fh, fw = w.shape
    assert ic == ic2
    oh, ow = conv_out(ih, fh, padding[0], stride[0], dilation[0]), conv_out(iw, fw, padding[1], stride[1], dilation[1])
    y = np.empty((bs, oc, oh, ow), dtype=np.float64)
    _lib.orc_conv2_naive_f64(_ptr(x), _ptr(w), _ptr(y), bs, ic, ih, iw, oc, fh, fw, padding[0], padding[1],
                             stride[0], stride[1], dilation[0], dilation[1])
    return y


def conv2_direct_f32(x, w):
    """Host f32 direct convolution, default options (stride 1, no padding, no dilation)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    bs, ic, ih, iw = x.shape
    oc, _, fh, fw = w.shape
    y = np.empty((bs, oc, ih - fh + 1, iw - fw + 1), dtype=np.float32)
    _lib.orc_conv2_direct_f32(_ptr(x), _ptr(w), _ptr(y), bs, ic, ih, iw, oc, fh, fw)
    return y


def conv2_direct_packed_f32(x, w, threads=0):
    """The reference host's f32 Conv2 for default options as it runs it (conv_direct.rs:84-96, :760-946): packed
    [f32; 8] layouts and a register-tiled AVX2/FMA kernel, images dealt to `threads` threads (0: all cores)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    bs, ic, ih, iw = x.shape
    oc, _, fh, fw = w.shape
    y = np.empty((bs, oc, ih - fh + 1, iw - fw + 1), dtype=np.float32)
    _lib.orc_conv2_direct_packed_f32(_ptr(x), _ptr(w), _ptr(y), bs, ic, ih, iw, oc, fh, fw, threads)
    return y


def lenet5_forward_f32(x, w1, w2, wd1, wd2, wd3, b3, threads=None, direct=False):
    """Weights: w1 [6,1,5,5], w2 [16,6,5,5], wd* [in,out] (Dense layout, layer.rs:482-486), b3 [10].
    direct=True runs the convolutions as a plain direct loop, direct="packed" (or 2) as the reference host runs
    them for f32 (conv_direct: packed layouts, register-tiled kernel)."""
    arrs = [np.ascontiguousarray(a, dtype=np.float32) for a in (x, w1, w2, wd1, wd2, wd3, b3)]
    bs = arrs[0].shape[0]
    out = np.empty((bs, 10), dtype=np.float32)
    _lib.orc_lenet5_forward_f32_alg(_ptr(arrs[0]), bs, *[_ptr(a) for a in arrs[1:]], _ptr(out),
                                    threads or min(4, max_threads()), 2 if direct in ("packed", 2) else (1 if direct else 0))
    return out


# ------------------------------------------------------------- training tail ----
def to_standard_layout(a):
    """Strided copy (<= 4-D) of any numpy view into a fresh C-contiguous array, through orc_assign4."""
    assert a.ndim <= 4
    es = a.itemsize
    base = a if a.base is None else a.base
    while base.base is not None:
        base = base.base
    base = np.asarray(base)
    off = (a.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // es
    pad = 4 - a.ndim
    dims = (C.c_int64 * 4)(*([1] * pad + list(a.shape)))
    sx = (C.c_int64 * 4)(*([0] * pad + [st // es for st in a.strides]))
    out = np.empty(a.shape, dtype=a.dtype)
    sy = (C.c_int64 * 4)(*([0] * pad + [st // es for st in out.strides]))
    _lib.orc_assign4(_ptr(base), off, sx, _ptr(out), 0, sy, dims, es)
    return out


def scaled_add(y, alpha, x):
    """y + alpha * x with the product and the sum each rounded to the element type; returns a new array."""
    y = np.array(y, order="C", copy=True)
    x = np.ascontiguousarray(x)
    assert x.shape == y.shape and x.dtype == y.dtype
    (_lib.orc_scaled_add_bf16 if _is_bf16(y) else _lib.orc_scaled_add_f32)(_ptr(y), float(alpha), _ptr(x), y.size)
    return y


def _base_off_strides(a):
    """(base array, element offset, element strides) of a numpy view."""
    base = a
    while base.base is not None and isinstance(base.base, np.ndarray):
        base = base.base
    es = a.dtype.itemsize
    off = (a.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // es
    return base, off, [st // es for st in a.strides]


def scaled_add_strided(y, alpha, x):
    """IN PLACE on the numpy view `y` (<= 4-D, any strides): y += alpha * broadcast(x), product and sum each rounded to
    the element type.  `x` is broadcast to y's shape as ndarray does (trailing axes aligned, stride 0)."""
    assert y.ndim <= 4 and x.dtype == y.dtype
    xb = np.broadcast_to(x, y.shape)
    pad = 4 - y.ndim
    yb, off_y, sy = _base_off_strides(y)
    xbase, off_x, sx = _base_off_strides(xb) if xb.base is not None else (xb, 0, [st // xb.itemsize for st in xb.strides])
    d = (C.c_int64 * 4)(*([1] * pad + list(y.shape)))
    sxa = (C.c_int64 * 4)(*([0] * pad + sx))
    sya = (C.c_int64 * 4)(*([0] * pad + sy))
    fn = _lib.orc_scaled_add_strided_bf16 if _is_bf16(y) else _lib.orc_scaled_add_strided_f32
    fn(_ptr(yb), off_y, sya, float(alpha), _ptr(xbase), off_x, sxa, d)
    return y


def accuracy(x, t):
    x, t = np.ascontiguousarray(x), np.ascontiguousarray(t, dtype=np.uint8)
    bs, classes = x.shape
    return int((_lib.orc_accuracy_bf16 if _is_bf16(x) else _lib.orc_accuracy_f32)(_ptr(x), _ptr(t), bs, classes))


def sgd_momentum(w, dw, lr, momentum, v):
    """Returns (w', v')."""
    w, v = np.array(w, order="C", copy=True), np.array(v, order="C", copy=True)
    dw = np.ascontiguousarray(dw)
    (_lib.orc_sgd_momentum_bf16 if _is_bf16(w) else _lib.orc_sgd_momentum_f32)(_ptr(w), _ptr(dw), float(lr), float(momentum), _ptr(v), w.size)
    return w, v


def sum_axis0(x):
    x = np.ascontiguousarray(x)
    rows, cols = x.shape
    y = np.empty(cols, dtype=x.dtype)
    (_lib.orc_sum_axis0_bf16 if _is_bf16(x) else _lib.orc_sum_axis0_f32)(_ptr(x), _ptr(y), rows, cols)
    return y


def cross_entropy_loss(x, t):
    x, t = np.ascontiguousarray(x), np.ascontiguousarray(t, dtype=np.uint8)
    bs, classes = x.shape
    return float((_lib.orc_cross_entropy_loss_bf16 if _is_bf16(x) else _lib.orc_cross_entropy_loss_f32)(_ptr(x), _ptr(t), bs, classes))


def cross_entropy_backward(x, t, dy=1.0):
    x, t = np.ascontiguousarray(x), np.ascontiguousarray(t, dtype=np.uint8)
    bs, classes = x.shape
    dx = np.empty_like(x)
    (_lib.orc_cross_entropy_backward_bf16 if _is_bf16(x) else _lib.orc_cross_entropy_backward_f32)(_ptr(x), _ptr(t), float(dy), _ptr(dx), bs, classes)
    return dx


def lenet5_train_step(x, t, params, lr=0.01, momentum=None, velocities=None, intermediates=None):
    """One training step of the benchmark's LeNet5 (benches/neural-network-benches/src/autograph_backend.rs:70-86,
    layers :88-162) chained from the host ops above in the order the autograd edges run them
    (layer.rs:950-1005 conv, autograd.rs:607-627 dot, :571-599 bias, layer.rs:1253-1267 relu, :1193-1216 pool).
    GEMMs use f32 accumulation with one rounding (the numerics the tolerance is stated against).
    params = [w1, w2, wd1, wd2, wd3, b3]; returns (loss, new_params, grads, new_velocities).  A dict passed as
    `intermediates` receives the masked gradients of the backward chain (g_logits, g_d2, g_d1, gm2, gm1)."""
    w1, w2, wd1, wd2, wd3, b3 = params
    bf = _is_bf16(w1)
    mm = gemm_bf16_f32acc if bf else (lambda a, b: gemm_f64acc(a, b).astype(np.float32))
    bs = x.shape[0]

    def conv_fwd(h, w):
        oc, ic, fh, fw = w.shape
        cols = im2col_conv2(h, (fh, fw))
        oh, ow = h.shape[2] - fh + 1, h.shape[3] - fw + 1
        ym = mm(cols, w.reshape(oc, -1).T)
        y = to_standard_layout(ym.reshape(bs, oh, ow, oc).transpose(0, 3, 1, 2))
        return cols, y

    cols1, c1 = conv_fwd(x, w1)
    r1 = relu(c1)
    p1 = max_pool2(r1, (2, 2))
    cols2, c2 = conv_fwd(p1, w2)
    r2 = relu(c2)
    p2 = max_pool2(r2, (2, 2))
    f = p2.reshape(bs, 256)
    d1 = mm(f, wd1)
    a1 = relu(d1)
    d2 = mm(a1, wd2)
    a2 = relu(d2)
    logits = bias_add_rows(mm(a2, wd3), b3)
    loss = cross_entropy_loss(logits, t)

    keep = intermediates if intermediates is not None else {}
    g = cross_entropy_backward(logits, t, 1.0)
    keep["g_logits"] = g
    db3 = sum_axis0(g)
    dwd3 = mm(a2.T, g)
    g = relu_backward(d2, mm(g, wd3.T))
    keep["g_d2"] = g
    dwd2 = mm(a1.T, g)
    g = relu_backward(d1, mm(g, wd2.T))
    keep["g_d1"] = g
    dwd1 = mm(f.T, g)
    g = mm(g, wd1.T).reshape(bs, 16, 4, 4)
    g = relu_backward(c2, max_pool2_backward(r2, g, (2, 2)))
    gm = to_standard_layout(g.transpose(0, 2, 3, 1)).reshape(bs * 64, 16)
    keep["gm2"] = gm
    dw2 = mm(gm.T, cols2).reshape(w2.shape)
    g = col2im_conv2(mm(gm, w2.reshape(16, 150)), (8, 8), (5, 5))
    g = relu_backward(c1, max_pool2_backward(r1, g, (2, 2)))
    gm = to_standard_layout(g.transpose(0, 2, 3, 1)).reshape(bs * 576, 6)
    keep["gm1"] = gm
    dw1 = mm(gm.T, cols1).reshape(w1.shape)

    grads = [dw1, dw2, dwd1, dwd2, dwd3, db3]
    if momentum is None:
        alpha = -lr
        new_params = [scaled_add(p, alpha, gr) for p, gr in zip(params, grads)]
        new_v = None
    else:
        if velocities is None:
            velocities = [np.zeros_like(p) for p in params]
        pairs = [sgd_momentum(p, gr, lr, momentum, v) for p, gr, v in zip(params, grads, velocities)]
        new_params, new_v = [a for a, _ in pairs], [b for _, b in pairs]
    return loss, new_params, grads, new_v
