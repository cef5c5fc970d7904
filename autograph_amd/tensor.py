"""Host-side mirror of the reference's tensor interface for the hot path.

`Device`, `Buffer` and `Tensor` carry exactly what the reference's device branches hand
to a kernel: a device allocation, an element offset, dims and signed element strides
(src/tensor.rs:327-332, :796-804).  Every operation below forwards to one C-ABI entry
point of libautograph_hip.so; nothing is computed on the host.

bf16 tensors travel as numpy ``uint16`` arrays of raw bit patterns.
"""
import contextlib
import ctypes as C
from dataclasses import dataclass, field
from typing import Tuple

import numpy as np

from ._ffi import AghError, check, lib

F32 = "f32"
BF16 = "bf16"
_ITEMSIZE = {F32: 4, BF16: 2}
_NPTYPE = {F32: np.float32, BF16: np.uint16}


def _dtype_of(array):
    if array.dtype == np.float32:
        return F32
    if array.dtype == np.uint16:
        return BF16
    raise TypeError(f"unsupported dtype {array.dtype}: use float32, or uint16 for bf16 bit patterns")


class Device:
    """`Device::builder().index(i).build()` (tests/integration_tests.rs:27-30)."""

    def __init__(self, index=0):
        check(lib.agh_init(index))
        self.index = index

    def info(self):
        name = C.create_string_buffer(256)
        cus = C.c_int()
        mem = C.c_size_t()
        check(lib.agh_device_info(name, 256, C.byref(cus), C.byref(mem)))
        return {"name": name.value.decode(), "compute_units": cus.value, "total_mem": mem.value}

    def wait(self):
        """`device.wait()` (src/tensor/linalg.rs:549)."""
        check(lib.agh_sync())


class Buffer:
    """Owning device allocation (krnl `Buffer`); freed when dropped."""

    def __init__(self, nbytes):
        p = C.c_void_p()
        check(lib.agh_malloc(C.byref(p), nbytes))
        self.ptr = p.value
        self.nbytes = nbytes

    def __del__(self):
        ptr, self.ptr = getattr(self, "ptr", None), None
        if ptr:
            try:
                lib.agh_free(ptr)
            except Exception:
                pass


# ---- option structs, src/ops.rs:9-108 ----
@dataclass
class Im2ColConv2Options:
    filter: Tuple[int, int] = (0, 0)
    padding: Tuple[int, int] = (0, 0)
    stride: Tuple[int, int] = (1, 1)
    dilation: Tuple[int, int] = (1, 1)

    def output_shape(self, input_shape):
        return tuple((a + 2 * p - d * (f - 1) - 1) // s + 1
                     for a, f, p, s, d in zip(input_shape, self.filter, self.padding, self.stride, self.dilation))


@dataclass
class Col2ImConv2Options:
    shape: Tuple[int, int] = (0, 0)
    filter: Tuple[int, int] = (0, 0)
    padding: Tuple[int, int] = (0, 0)
    stride: Tuple[int, int] = (1, 1)
    dilation: Tuple[int, int] = (1, 1)

    def output_shape(self):
        return tuple((a - 1) * s + d * (f - 1) + 1 - 2 * p
                     for a, f, p, s, d in zip(self.shape, self.filter, self.padding, self.stride, self.dilation))


@dataclass
class MaxPool2Options:
    size: Tuple[int, int] = (2, 2)
    strides: Tuple[int, int] = (2, 2)

    def output_shape(self, input_shape):
        return tuple((a - x) // s + 1 for a, x, s in zip(input_shape, self.size, self.strides))


def _std_strides(shape):
    strides, acc = [], 1
    for d in reversed(shape):
        strides.append(acc)
        acc *= d
    return tuple(reversed(strides))


class Tensor:
    """`TensorBase` = {dim, strides, buffer, offset} (src/tensor.rs:327-332) on the device."""

    def __init__(self, buffer, shape, strides, offset, dtype):
        self.buffer, self.shape, self.strides, self.offset, self.dtype = buffer, tuple(shape), tuple(strides), offset, dtype

    # -- construction / transfer (src/tensor.rs:1377-1416, :1775-1833, :1923-1934) --
    @classmethod
    def uninit(cls, shape, dtype):
        n = int(np.prod(shape)) if len(shape) else 1
        return cls(Buffer(n * _ITEMSIZE[dtype]), shape, _std_strides(shape), 0, dtype)

    @classmethod
    def zeros(cls, shape, dtype):
        t = cls.uninit(shape, dtype)
        check(lib.agh_memset(t.buffer.ptr, 0, t.buffer.nbytes))
        return t

    @classmethod
    def from_array(cls, array):
        """`Tensor::from(array).into_device(device)`: copies in standard layout."""
        a = np.ascontiguousarray(array)
        t = cls.uninit(a.shape, _dtype_of(a))
        check(lib.agh_memcpy_h2d(t.buffer.ptr, a.ctypes.data, a.nbytes))
        check(lib.agh_sync())  # `a` may be a temporary
        return t

    # -- serde (src/tensor.rs:1199-1249): the reference's data model, as serde_json writes it --
    def to_json(self):
        """Blocking: copies the data to the host (standard layout) and encodes them; see autograph_amd/serde.py."""
        from . import serde
        return serde.to_json(self.into_array(), bf16=self.dtype == "bf16")

    @classmethod
    def from_json(cls, text, dtype=None):
        """Decodes a tensor the reference (or `to_json`) wrote and uploads it.  `dtype` ("f32" / "bf16"), when
        given, must match what the text holds, as the typed `Tensor<T, D>` deserialiser's conversion would."""
        from . import serde
        array, is_bf16 = serde.from_json(text)
        if not is_bf16 and array.dtype != np.float32:
            raise AghError(-1, f"serde: scalar type {serde.scalar_name(array)} has no device tensor here (f32 and bf16 only)")
        got = "bf16" if is_bf16 else "f32"
        if dtype is not None and dtype != got:
            raise AghError(-1, f"Expected {dtype} found {got}")
        return cls.from_array(array)

    def into_array(self):
        """`into_array()`: blocking copy of the whole buffer, then the same strided view."""
        raw = np.empty(self.buffer.nbytes // _ITEMSIZE[self.dtype], dtype=_NPTYPE[self.dtype])
        check(lib.agh_memcpy_d2h(raw.ctypes.data, self.buffer.ptr, self.buffer.nbytes))
        es = raw.itemsize
        view = np.lib.stride_tricks.as_strided(raw[self.offset:], shape=self.shape,
                                               strides=tuple(s * es for s in self.strides))
        return np.array(view, order="C", copy=True)

    # -- views (src/tensor.rs:695-703, :103-122) --
    @property
    def ndim(self):
        return len(self.shape)

    def __len__(self):
        return int(np.prod(self.shape))

    def is_standard_layout(self):
        return all(d == 1 or s == e for d, s, e in zip(self.shape, self.strides, _std_strides(self.shape)))

    def t(self):
        return Tensor(self.buffer, self.shape[::-1], self.strides[::-1], self.offset, self.dtype)

    def permuted_axes(self, axes):
        return Tensor(self.buffer, [self.shape[a] for a in axes], [self.strides[a] for a in axes], self.offset, self.dtype)

    def into_shape(self, shape):
        if not self.is_standard_layout():
            raise AghError(-1, "into_shape: tensor is not in standard layout")  # tensor.rs:103-122
        if int(np.prod(shape)) != len(self):
            raise AghError(-1, f"into_shape: incompatible shapes {self.shape} -> {tuple(shape)}")
        return Tensor(self.buffer, shape, _std_strides(shape), self.offset, self.dtype)

    def slice_rows(self, start, stop, step=1):
        """Row slice of a 2-D tensor; a negative step gives the negative-stride views ndarray allows."""
        assert self.ndim == 2
        idx = range(self.shape[0])[start:stop:step]
        off = self.offset + (idx.start if len(idx) else 0) * self.strides[0]
        return Tensor(self.buffer, (len(idx), self.shape[1]), (self.strides[0] * step, self.strides[1]), off, self.dtype)

    def _ptr(self):
        return self.buffer.ptr

    def _fn(self, stem):
        return getattr(lib, f"{stem}_{self.dtype}")

    # -- Dot, src/tensor/linalg.rs:362-468 --
    def dot(self, rhs, bias=None, relu=False):
        """`self.dot(&rhs)`; with `bias`/`relu` the Dense epilogue is fused into the same launch."""
        if self.dtype != rhs.dtype:
            raise AghError(-1, f"Can not dot tensors of different types {self.dtype} != {rhs.dtype}!")  # linalg.rs:428-434
        if self.ndim != 2 or rhs.ndim != 2:
            raise AghError(-1, "dot: both operands must be 2-D")
        m, k = self.shape
        k2, n = rhs.shape
        if k != k2:
            raise AghError(-1, f"a_cols != b_rows, {k} != {k2}")  # linalg.rs:274-276
        out = Tensor.uninit((m, n), self.dtype)
        gemm(1.0, self, rhs, 0.0, out, bias=bias, relu=relu)
        return out

    # -- Im2ColConv2 / Col2ImConv2, src/tensor/ops.rs:831-888, :982-1037 --
    def im2col_conv2(self, options):
        x = self.as_standard_layout()
        bs, c, ih, iw = x.shape
        oh, ow = options.output_shape((ih, iw))
        (fh, fw), (ph, pw), (sh, sw), (dh, dw) = options.filter, options.padding, options.stride, options.dilation
        y = Tensor.uninit((bs * oh * ow, c * fh * fw), self.dtype)
        check(self._fn("agh_im2col_conv2")(x._data_ptr(), y._ptr(), bs, c, ih, iw, fh, fw, ph, pw, sh, sw, dh, dw))
        return y

    def col2im_conv2(self, options):
        x = self.as_standard_layout()
        rows, cols = x.shape
        ih, iw = options.shape
        (fh, fw), (ph, pw), (sh, sw), (dh, dw) = options.filter, options.padding, options.stride, options.dilation
        bs, c = rows // (ih * iw), cols // (fh * fw)
        oh, ow = options.output_shape()
        y = Tensor.uninit((bs, c, oh, ow), self.dtype)
        check(self._fn("agh_col2im_conv2")(x._data_ptr(), y._ptr(), bs, c, ih, iw, fh, fw, ph, pw, sh, sw, dh, dw))
        return y

    # -- MaxPool2 / MaxPool2Backward, src/tensor/ops.rs:1106-1141, :1228-1275 --
    def max_pool2(self, options):
        x = self.as_standard_layout()
        bs, c, ih, iw = x.shape
        oh, ow = options.output_shape((ih, iw))
        y = Tensor.uninit((bs, c, oh, ow), self.dtype)
        check(self._fn("agh_max_pool2")(x._data_ptr(), y._ptr(), bs * c, ih, iw, *options.size, *options.strides))
        return y

    def max_pool2_backward(self, output_grad, options):
        """In place: `self` holds x on entry and dx on return (layer.rs:1203-1211 clones x first)."""
        if self.dtype != output_grad.dtype:
            raise AghError(-1, f"Expected {self.dtype} found {output_grad.dtype}")  # ops.rs:1236-1242
        if not self.is_standard_layout():
            raise AghError(-1, "max_pool2_backward: input gradient must be in standard layout")
        dy = output_grad.as_standard_layout()
        bs, c, ih, iw = self.shape
        check(self._fn("agh_max_pool2_backward")(self._data_ptr(), dy._data_ptr(), bs * c, ih, iw,
                                                 *options.size, *options.strides))

    # -- relu, layer.rs:1269-1510 --
    def relu(self):
        x = self.as_standard_layout()
        y = Tensor.uninit(x.shape, x.dtype)
        check(self._fn("agh_relu")(x._data_ptr(), y._ptr(), len(x)))
        return y

    def relu_backward(self, output_grad):
        x, dy = self.as_standard_layout(), output_grad.as_standard_layout()
        dx = Tensor.uninit(x.shape, x.dtype)
        check(self._fn("agh_relu_backward")(x._data_ptr(), dy._data_ptr(), dx._ptr(), len(x)))
        return dx

    # -- helpers --
    def _data_ptr(self):
        return self.buffer.ptr + self.offset * _ITEMSIZE[self.dtype]

    def clone(self):
        assert self.is_standard_layout()
        out = Tensor.uninit(self.shape, self.dtype)
        check(lib.agh_memcpy_d2d(out._ptr(), self._data_ptr(), len(self) * _ITEMSIZE[self.dtype]))
        return out

    def as_standard_layout(self):
        """`as_standard_layout` (src/tensor.rs): self if already contiguous, else a strided copy."""
        if self.is_standard_layout():
            return self
        return self.to_standard_layout()

    def to_standard_layout(self):
        """Strided copy into a fresh standard-layout tensor (`assign`, src/tensor/ops.rs:257-318)."""
        if self.ndim > 4:
            raise AghError(-1, "to_standard_layout: more than 4 dimensions")
        out = Tensor.uninit(self.shape, self.dtype)
        pad = 4 - self.ndim
        dims = [1] * pad + list(self.shape)
        sx = [0] * pad + list(self.strides)
        sy = [0] * pad + list(out.strides)
        check(self._fn("agh_assign")(self._ptr(), self.offset, *sx, out._ptr(), 0, *sy, *dims))
        return out

    def broadcast(self, shape):
        """View with stride 0 along broadcast axes (ndarray `broadcast`)."""
        shape = tuple(shape)
        pad = len(shape) - self.ndim
        if pad < 0:
            return None
        strides = [0] * pad
        for d, s, want in zip(self.shape, self.strides, shape[pad:]):
            if d == want:
                strides.append(s)
            elif d == 1:
                strides.append(0)
            else:
                return None
        return Tensor(self.buffer, shape, strides, self.offset, self.dtype)

    # -- scaled_add / sum_axis / cross entropy (src/tensor/ops.rs:257-318, reduce.rs:59-113, learn/criterion.rs) --
    def scaled_add(self, alpha, rhs):
        """In place: self += alpha * rhs with `rhs` broadcast to self's shape, the product and the sum each rounded to
        the element type (src/tensor/ops.rs:192-204 -> `assign(BinaryOp::Add, ..)`, :257-318).  Both sides may be any
        views of up to four dimensions."""
        if self.dtype != rhs.dtype:
            raise AghError(-1, f"scaled_add: {self.dtype} vs {rhs.dtype}")
        x = rhs.broadcast(self.shape)
        if x is None:
            raise AghError(-1, f"Broadcast not possible! {rhs.shape} -> {self.shape}")  # ops.rs:287-291
        if self.is_standard_layout() and x.is_standard_layout() and x.shape == rhs.shape:
            check(self._fn("agh_scaled_add")(self._data_ptr(), alpha, x._data_ptr(), len(self)))
            return
        if self.ndim > 4:
            raise AghError(-1, "scaled_add: more than 4 dimensions")
        pad = 4 - self.ndim
        dims = [1] * pad + list(self.shape)
        sy = [0] * pad + list(self.strides)
        sx = [0] * pad + list(x.strides)
        check(self._fn("agh_scaled_add_strided")(self._ptr(), self.offset, *sy, alpha, x._ptr(), x.offset, *sx, *dims))

    def add_assign(self, rhs):
        """`AddAssign` (src/tensor/ops.rs:245-255): `self.scaled_add(T::one(), &rhs)`."""
        self.scaled_add(1.0, rhs)

    def accuracy(self, target):
        """`Accuracy::accuracy` (src/learn/criterion.rs:22-118): the number of rows whose target class has the strictly
        largest score.  `target`: u8 class indices on the device (a `Buffer`).  Blocking."""
        x = self.as_standard_layout()
        bs, classes = x.shape
        tmp = Buffer(4)
        check(self._fn("agh_accuracy")(x._data_ptr(), target.ptr, bs, classes, tmp.ptr))
        out = np.empty(1, dtype=np.uint32)
        check(lib.agh_memcpy_d2h(out.ctypes.data, tmp.ptr, 4))
        return int(out[0])

    def sum_axis0(self):
        x = self.as_standard_layout()
        rows, cols = x.shape
        y = Tensor.uninit((cols,), self.dtype)
        check(self._fn("agh_sum_axis0")(x._data_ptr(), y._ptr(), rows, cols))
        return y

    def cross_entropy_loss(self, target, out_ptr=None):
        """Sum of the per-row losses (f32).  `target`: u8 class indices on the device (a `Buffer`).
        With `out_ptr` (device or pinned host memory) nothing is copied back and None is returned."""
        x = self.as_standard_layout()
        bs, classes = x.shape
        if out_ptr is not None:
            check(self._fn("agh_cross_entropy_loss")(x._data_ptr(), target.ptr, bs, classes, out_ptr))
            return None
        tmp = Buffer(4)
        check(self._fn("agh_cross_entropy_loss")(x._data_ptr(), target.ptr, bs, classes, tmp.ptr))
        out = np.empty(1, dtype=np.float32)
        check(lib.agh_memcpy_d2h(out.ctypes.data, tmp.ptr, 4))
        return float(out[0])

    def cross_entropy_loss_backward(self, target, dy=1.0):
        x = self.as_standard_layout()
        bs, classes = x.shape
        dx = Tensor.uninit(x.shape, x.dtype)
        check(self._fn("agh_cross_entropy_backward")(x._data_ptr(), target.ptr, dy, dx._ptr(), bs, classes))
        return dx


@contextlib.contextmanager
def branch():
    """Work issued inside the block goes to the library's second stream: it starts after everything
    issued before the block and runs beside what follows it, until `join()`.  The caller vouches that
    the two sides write disjoint memory."""
    check(lib.agh_branch_begin())
    try:
        yield
    finally:
        check(lib.agh_branch_end())


def join():
    """Later work waits for every `branch()` issued so far."""
    check(lib.agh_branch_join())


def gemm(alpha, a, b, beta, c, bias=None, relu=False):
    """`fn gemm(alpha, a, b, beta, c)` with the reference's checks (src/tensor/linalg.rs:249-299)."""
    if a.dtype != b.dtype:
        raise AghError(-1, f"a_scalar_type != b_scalar_type, {a.dtype} != {b.dtype}")
    if a.dtype != c.dtype:
        raise AghError(-1, f"a_scalar_type != c_scalar_type, {a.dtype} != {c.dtype}")
    (m, k), (k2, n), (m2, n2) = a.shape, b.shape, c.shape
    if m != m2:
        raise AghError(-1, f"a_rows != c_rows, {m} != {m2}")
    if k != k2:
        raise AghError(-1, f"a_cols != b_rows, {k} != {k2}")
    if n != n2:
        raise AghError(-1, f"b_cols != c_rows, {n} != {n2}")
    common = (m, k, n, alpha, a._ptr(), a.offset, a.strides[0], a.strides[1], b._ptr(), b.offset, b.strides[0],
              b.strides[1], beta, c._ptr(), c.offset, c.strides[0], c.strides[1])
    if bias is None and not relu:
        check(getattr(lib, f"agh_gemm_{c.dtype}")(*common))
    else:
        if bias is not None and (bias.dtype != c.dtype or bias.shape != (n,)):
            raise AghError(-1, f"bias must be a {c.dtype} vector of length {n}")
        bp, bo, bs_ = (bias._ptr(), bias.offset, bias.strides[0]) if bias is not None else (None, 0, 0)
        check(getattr(lib, f"agh_gemm_{c.dtype}_bias_act")(*common, bp, bo, bs_, 1 if relu else 0))
