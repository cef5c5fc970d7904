"""Host-side mirror of the reference's layer structs for the hot path:
`Conv2`, `Dense`, `MaxPool2`, `Relu`, `Flatten` with `forward` (src/learn/neural_network/layer.rs),
and the LeNet5 model of the reference's benchmark (benches/neural-network-benches/src/
autograph_backend.rs:88-162).  Inference only: parameters are plain tensors.
"""
import ctypes as C

import numpy as np

from ._ffi import AghError, check, lib
from .tensor import Im2ColConv2Options, MaxPool2Options, Tensor, _ITEMSIZE


def conv2_im2col_forward(x, weight, padding=(0, 0), stride=(1, 1), dilation=(1, 1), bias=None, relu=False):
    """`conv2_im2col` (layer.rs:950-1005): im2col, dot with the [oc, ic*fh*fw] weight matrix
    transposed, result in NCHW.  The NHWC->NCHW copy of the reference is folded into the GEMM:
    per image the [oh*ow, oc] product is written column-major, which IS the NCHW plane order."""
    bs, ic, ih, iw = x.shape
    oc, ic2, fh, fw = weight.shape
    if ic != ic2:
        raise AghError(-1, f"conv2: input has {ic} channels, weight expects {ic2}")
    opts = Im2ColConv2Options(filter=(fh, fw), padding=tuple(padding), stride=tuple(stride), dilation=tuple(dilation))
    oh, ow = opts.output_shape((ih, iw))
    cols = x.im2col_conv2(opts)                      # [bs*oh*ow, ic*fh*fw]
    wm = weight.into_shape((oc, ic * fh * fw))       # view, no copy
    y = Tensor.uninit((bs, oc, oh, ow), x.dtype)
    L, K = oh * ow, ic * fh * fw
    bp, bo, bst = (bias._ptr(), bias.offset, bias.strides[0]) if bias is not None else (None, 0, 0)
    # A_b = cols[b*L:(b+1)*L, :], B = wm^T (rsb = 1, csb = K), C_b[hw, o] at y + b*oc*L + o*L + hw
    check(getattr(lib, f"agh_gemm_{x.dtype}_batched")(
        bs, L, K, oc, 1.0, cols._ptr(), cols.offset, K, 1, L * K, wm._ptr(), wm.offset, 1, K, 0,
        0.0, y._ptr(), y.offset, 1, L, oc * L, bp, bo, bst, 1 if relu else 0))
    return y


def conv2_direct_forward(x, weight, padding=(0, 0), stride=(1, 1), dilation=(1, 1), bias=None, relu=False, pool2x2=False):
    """Direct convolution out of LDS (agh_conv2_direct_*), optionally with the following Relu and
    2x2/2 MaxPool2 fused.  Raises AghError(AGH_ERANGE) when the layer does not fit in LDS."""
    x = x.as_standard_layout()
    bs, ic, ih, iw = x.shape
    oc, ic2, fh, fw = weight.shape
    if ic != ic2:
        raise AghError(-1, f"conv2: input has {ic} channels, weight expects {ic2}")
    opts = Im2ColConv2Options(filter=(fh, fw), padding=tuple(padding), stride=tuple(stride), dilation=tuple(dilation))
    oh, ow = opts.output_shape((ih, iw))
    yshape = (bs, oc, oh // 2, ow // 2) if pool2x2 else (bs, oc, oh, ow)
    y = Tensor.uninit(yshape, x.dtype)
    check(getattr(lib, f"agh_conv2_direct_{x.dtype}")(
        x._data_ptr(), weight.as_standard_layout()._data_ptr(), bias._data_ptr() if bias is not None else None,
        y._ptr(), bs, ic, ih, iw, oc, fh, fw, *padding, *stride, *dilation, 1 if relu else 0, 1 if pool2x2 else 0))
    return y


class Conv2:
    """`Conv2` (layer.rs:844-1047): weight [outputs, inputs, fh, fw], optional bias [outputs]."""

    def __init__(self, weight, bias=None, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
        self.weight, self.bias = weight, bias
        self.padding, self.stride, self.dilation = tuple(padding), tuple(stride), tuple(dilation)

    def forward(self, x, relu=False, pool2x2=False, algorithm="auto"):
        """`conv2` (layer.rs:930-948).  Like the reference's host, which takes a direct kernel when
        it can and im2col otherwise, `auto` tries the LDS-resident direct kernel first."""
        kw = dict(padding=self.padding, stride=self.stride, dilation=self.dilation, bias=self.bias)
        if algorithm in ("auto", "direct"):
            try:
                return conv2_direct_forward(x, self.weight, relu=relu, pool2x2=pool2x2, **kw)
            except AghError as e:
                if algorithm == "direct" or e.code != -4:
                    raise
        y = conv2_im2col_forward(x, self.weight, relu=relu, **kw)
        if pool2x2:
            y = y.max_pool2(MaxPool2Options((2, 2), (2, 2)))
        return y


class Dense:
    """`Dense` (layer.rs:1050-1143): weight [inputs, outputs], optional bias [outputs]."""

    def __init__(self, weight, bias=None):
        self.weight, self.bias = weight, bias

    def forward(self, x, relu=False):
        return x.dot(self.weight, bias=self.bias, relu=relu)


class MaxPool2:
    """`MaxPool2` (layer.rs:1149-1216); stride defaults to the filter (layer.rs:535-539)."""

    def __init__(self, filter, stride=None):
        self.filter = tuple(filter)
        self.stride = tuple(stride) if stride is not None else self.filter

    def forward(self, x):
        return x.max_pool2(MaxPool2Options(self.filter, self.stride))


class Relu:
    def forward(self, x):
        return x.relu()


class Flatten:
    def forward(self, x):
        return x.into_shape((x.shape[0], int(np.prod(x.shape[1:]))))


class LeNet5:
    """conv 1->6 5x5, relu, pool 2x2, conv 6->16 5x5, relu, pool 2x2, flatten, dense 256->128, relu,
    dense 128->84, relu, dense 84->10 with bias (autograph_backend.rs:88-162)."""

    def __init__(self, w1, w2, wd1, wd2, wd3, b3):
        self.conv1, self.conv2 = Conv2(w1), Conv2(w2)
        self.pool = MaxPool2((2, 2))
        self.relu, self.flatten = Relu(), Flatten()
        self.dense1, self.dense2, self.dense3 = Dense(wd1), Dense(wd2), Dense(wd3, b3)
        self._graph = None

    @classmethod
    def from_arrays(cls, *arrays):
        return cls(*[Tensor.from_array(a) for a in arrays])

    def forward(self, x, algorithm="im2col"):
        """Layer by layer, twelve launches, exactly the structure `#[derive(Forward)]` expands to."""
        h = self.pool.forward(self.relu.forward(self.conv1.forward(x, algorithm=algorithm)))
        h = self.pool.forward(self.relu.forward(self.conv2.forward(h, algorithm=algorithm)))
        h = self.flatten.forward(h)
        h = self.relu.forward(self.dense1.forward(h))
        h = self.relu.forward(self.dense2.forward(h))
        return self.dense3.forward(h)

    def forward_fused(self, x):
        """Same results per layer, five launches: each conv with its Relu and MaxPool2 fused,
        each Dense with its bias/Relu in the GEMM epilogue."""
        h = self.conv1.forward(x, relu=True, pool2x2=True)
        h = self.conv2.forward(h, relu=True, pool2x2=True)
        h = self.flatten.forward(h)
        h = self.dense1.forward(h, relu=True)
        h = self.dense2.forward(h, relu=True)
        return self.dense3.forward(h)

    def forward_single_launch(self, x, out_ptr=None):
        """The whole forward pass as ONE kernel (agh_lenet5_forward_*), activations in LDS.  With
        `out_ptr` (device memory or pinned host memory) the logits go there; else a new tensor."""
        x = x.as_standard_layout()
        bs = x.shape[0]
        if x.shape[1:] != (1, 28, 28):
            raise AghError(-1, f"LeNet5 expects [bs,1,28,28] inputs, got {x.shape}")
        out = None
        if out_ptr is None:
            out = Tensor.uninit((bs, 10), x.dtype)
            out_ptr = out._ptr()
        ws = [self.conv1.weight, self.conv2.weight, self.dense1.weight, self.dense2.weight, self.dense3.weight,
              self.dense3.bias]
        check(getattr(lib, f"agh_lenet5_forward_{x.dtype}")(x._data_ptr(), *[w.as_standard_layout()._data_ptr() for w in ws],
                                                           out_ptr, bs))
        return out

    # -- graph-captured inference on fixed buffers --
    def capture(self, x, host_out_ptr=None):
        """Record `forward_fused` on `x` (and, if given, the device->host copy of the logits into a
        pinned host buffer) into a hipGraph.  Intermediates are allocated once here and reused by
        every replay; returns the logits tensor."""
        bs = x.shape[0]
        dt = x.dtype
        self._bufs = [Tensor.uninit(s, dt) for s in ((bs, 6, 12, 12), (bs, 16, 4, 4), (bs, 128), (bs, 84), (bs, 10))]
        self._run(x)  # eager warm-up: everything that allocates happens here
        check(lib.agh_sync())
        check(lib.agh_graph_begin())
        try:
            self._run(x)
            if host_out_ptr is not None:
                out = self._bufs[4]
                check(lib.agh_memcpy_d2h_async(host_out_ptr, out._ptr(), len(out) * _ITEMSIZE[dt]))
        finally:
            g = C.c_void_p()
            check(lib.agh_graph_end(C.byref(g)))
        self._graph = g
        return self._bufs[4]

    def _run(self, x):
        p1, p2, d1, d2, out = self._bufs
        dt = x.dtype
        bs = x.shape[0]
        conv = getattr(lib, f"agh_conv2_direct_{dt}")
        gemm = getattr(lib, f"agh_gemm_{dt}_bias_act")
        check(conv(x._data_ptr(), self.conv1.weight._data_ptr(), None, p1._ptr(), bs, 1, 28, 28, 6, 5, 5, 0, 0, 1, 1, 1, 1, 1, 1))
        check(conv(p1._ptr(), self.conv2.weight._data_ptr(), None, p2._ptr(), bs, 6, 12, 12, 16, 5, 5, 0, 0, 1, 1, 1, 1, 1, 1))
        w1, w2, w3, b3 = self.dense1.weight, self.dense2.weight, self.dense3.weight, self.dense3.bias
        check(gemm(bs, 256, 128, 1.0, p2._ptr(), 0, 256, 1, w1._ptr(), w1.offset, 128, 1, 0.0, d1._ptr(), 0, 128, 1, None, 0, 0, 1))
        check(gemm(bs, 128, 84, 1.0, d1._ptr(), 0, 128, 1, w2._ptr(), w2.offset, 84, 1, 0.0, d2._ptr(), 0, 84, 1, None, 0, 0, 1))
        check(gemm(bs, 84, 10, 1.0, d2._ptr(), 0, 84, 1, w3._ptr(), w3.offset, 10, 1, 0.0, out._ptr(), 0, 10, 1,
                   b3._ptr(), b3.offset, b3.strides[0], 0))

    def replay(self):
        check(lib.agh_graph_launch(self._graph))

    def __del__(self):
        g, self._graph = getattr(self, "_graph", None), None
        if g:
            try:
                lib.agh_graph_destroy(g)
            except Exception:
                pass
