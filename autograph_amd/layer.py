"""Host-side mirror of the reference's layer structs for the hot path:
`Conv2`, `Dense`, `MaxPool2`, `Relu`, `Flatten` with `forward` (src/learn/neural_network/layer.rs),
and the LeNet5 model of the reference's benchmark (benches/neural-network-benches/src/
autograph_backend.rs:88-162), plus one training step of it (`LeNet5Trainer`, `SGD`).
"""
import contextlib
import ctypes as C

import numpy as np

from ._ffi import AghError, check, lib
from .tensor import Im2ColConv2Options, MaxPool2Options, Tensor, _ITEMSIZE, _std_strides, branch, gemm, join


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
    # standard-layout copies of strided views are bound to names: they must outlive the launch call
    w = weight.as_standard_layout()
    b = bias.as_standard_layout() if bias is not None else None
    check(getattr(lib, f"agh_conv2_direct_{x.dtype}")(
        x._data_ptr(), w._data_ptr(), b._data_ptr() if b is not None else None,
        y._ptr(), bs, ic, ih, iw, oc, fh, fw, *padding, *stride, *dilation, 1 if relu else 0, 1 if pool2x2 else 0))
    return y


def _device_param(pair, dtype):
    """(array, is_bf16) of autograph_amd.serde -> device tensor, checked against an expected element type"""
    if pair is None:
        return None
    array, is_bf16 = pair
    got = "bf16" if is_bf16 else "f32"
    if not is_bf16 and array.dtype != np.float32:
        raise AghError(-1, "serde: parameters are f32 or bf16 here")
    if dtype is not None and dtype != got:
        raise AghError(-1, f"Expected {dtype} found {got}")
    return Tensor.from_array(array)


class OptimizerState:
    """`State` of a parameter (optimizer.rs:163-173) with its tensors on the device: `name` of the optimizer and
    `key_values` [(key, Tensor, parameter_device, parameter_type)].  A state read back from JSON is kept and written
    again, but an optimizer starts a fresh one: the reference skips the optimizer's type id when it writes a state and
    restores `()`'s (optimizer.rs:169-170, :175-178), which `SGD::init_state` then takes for another optimizer's state
    and replaces with a zero velocity (optimizer.rs:358-381)."""

    def __init__(self, name, key_values=()):
        self.name, self.key_values = name, list(key_values)

    def get(self, key):
        for k, t, _, _ in self.key_values:
            if k == key:
                return t
        return None


def _host_state(state):
    from . import serde
    if state is None:
        return None
    return serde.OptimStateValue(state.name, [(k, t.into_array(), t.dtype == "bf16", pd, pt) for k, t, pd, pt in state.key_values])


def _device_state(pair):
    st = getattr(pair, "optim_state", None)
    if st is None:
        return None
    for _, array, is_bf16, _, _ in st.key_values:
        if not is_bf16 and array.dtype != np.float32:
            raise AghError(-1, "serde: optimizer state tensors are f32 or bf16 here")
    return OptimizerState(st.name, [(k, Tensor.from_array(a), pd, pt) for k, a, _, pd, pt in st.key_values])


class Conv2:
    """`Conv2` (layer.rs:844-1047): weight [outputs, inputs, fh, fw], optional bias [outputs]."""

    def __init__(self, weight, bias=None, padding=(0, 0), stride=(1, 1), dilation=(1, 1)):
        self.weight, self.bias = weight, bias
        self.padding, self.stride, self.dilation = tuple(padding), tuple(stride), tuple(dilation)
        self.weight_state = self.bias_state = None  # OptimizerState of each parameter (autograd.rs:655)

    # the data model of the reference's derive (layer.rs:833-848), as serde_json writes it; see autograph_amd/serde.py
    def to_json(self):
        import json
        from . import serde
        bf16 = self.weight.dtype == "bf16"
        return json.dumps(serde.conv2_to_value(self.weight.into_array(), None if self.bias is None else self.bias.into_array(),
                                               self.padding, self.stride, self.dilation, bf16=bf16,
                                               weight_state=_host_state(self.weight_state),
                                               bias_state=_host_state(self.bias_state)), separators=(",", ":"))

    @classmethod
    def from_json(cls, text, dtype=None):
        import json
        from . import serde
        f = serde.conv2_from_value(json.loads(text))
        layer = cls(_device_param(f["weight"], dtype), _device_param(f["bias"], dtype), f["padding"], f["stride"], f["dilation"])
        layer.weight_state, layer.bias_state = _device_state(f["weight"]), _device_state(f["bias"])
        return layer

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
        self.weight_state = self.bias_state = None  # OptimizerState of each parameter (autograd.rs:655)

    def forward(self, x, relu=False, fused=True):
        """`Dense::forward` (layer.rs:1134-1143): `input.dot(&weight)` then `output.add_assign(&bias)`, and the Relu
        layer behind it when `relu`.  fused (default): one launch, bias and relu in the GEMM epilogue; fused=False runs
        the reference's separate calls (dot, broadcast add_assign, relu), bit-identical to the fused launch."""
        if fused:
            return x.dot(self.weight, bias=self.bias, relu=relu)
        out = x.dot(self.weight)
        if self.bias is not None:
            out.add_assign(self.bias)
        return out.relu() if relu else out

    def to_json(self):
        import json
        from . import serde
        return json.dumps(serde.dense_to_value(self.weight.into_array(), None if self.bias is None else self.bias.into_array(),
                                               bf16=self.weight.dtype == "bf16", weight_state=_host_state(self.weight_state),
                                               bias_state=_host_state(self.bias_state)), separators=(",", ":"))

    @classmethod
    def from_json(cls, text, dtype=None):
        import json
        from . import serde
        f = serde.dense_from_value(json.loads(text))
        layer = cls(_device_param(f["weight"], dtype), _device_param(f["bias"], dtype))
        layer.weight_state, layer.bias_state = _device_state(f["weight"]), _device_state(f["bias"])
        return layer


class MaxPool2:
    """`MaxPool2` (layer.rs:1149-1216); stride defaults to the filter (layer.rs:535-539)."""

    def __init__(self, filter, stride=None):
        self.filter = tuple(filter)
        self.stride = tuple(stride) if stride is not None else self.filter

    def forward(self, x):
        return x.max_pool2(MaxPool2Options(self.filter, self.stride))

    def to_json(self):
        import json
        from . import serde
        return json.dumps(serde.max_pool2_to_value(self.filter, self.stride), separators=(",", ":"))

    @classmethod
    def from_json(cls, text):
        import json
        from . import serde
        return cls(**serde.max_pool2_from_value(json.loads(text)))


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
        # standard-layout copies of strided views stay referenced by `ws` until the launch call has returned
        ws = [w.as_standard_layout() for w in (self.conv1.weight, self.conv2.weight, self.dense1.weight, self.dense2.weight,
                                               self.dense3.weight, self.dense3.bias)]
        check(getattr(lib, f"agh_lenet5_forward_{x.dtype}")(x._data_ptr(), *[w._data_ptr() for w in ws], out_ptr, bs))
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
        for t in (x, self.conv1.weight, self.conv2.weight):
            if not t.is_standard_layout():  # raw pointers below: a captured graph cannot own a copy
                raise AghError(-1, "LeNet5.capture: input and convolution weights must be in standard layout")
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


class SGD:
    """`SGD` (optimizer.rs:389-427): plain `scaled_add(-learning_rate)` or, with momentum, the f32
    velocity update of optimizer.rs:509-512."""

    def __init__(self, momentum=None):
        self.momentum = momentum

    def update(self, learning_rate, value, grad, velocity=None):
        if self.momentum is None:
            check(getattr(lib, f"agh_scaled_add_{value.dtype}")(value._data_ptr(), -learning_rate, grad._data_ptr(), len(value)))
        else:
            check(getattr(lib, f"agh_sgd_momentum_{value.dtype}")(value._data_ptr(), grad._data_ptr(), learning_rate,
                                                                  self.momentum, velocity._data_ptr(), len(value)))


class LeNet5Trainer:
    """One training step of the benchmark's LeNet5 (autograph_backend.rs:70-86): forward, summed
    cross-entropy loss, backward through the edges the reference's autograd builds (conv:
    layer.rs:950-1005, dot: autograd.rs:607-627, bias: :571-599 and :490-542, relu: layer.rs:1253-1267,
    pool: layer.rs:1193-1216, flatten / permute: autograd.rs:384-445), and the SGD update.

    Every buffer is allocated here, once; `step` only launches kernels, so it can be captured into
    a graph (`capture`) and replayed.  Gradients stay available in `grads` after a step.  `overlap`
    issues the weight gradients beside the input-gradient chain (`branch`); same kernels, same bits."""

    def __init__(self, model, batch_size, learning_rate=0.01, optimizer=None, overlap=None, fused_forward=None,
                 fused_backward=True):
        self.model, self.bs, self.lr = model, batch_size, learning_rate
        # fused_forward: the forward pass is ONE launch (agh_lenet5_forward_train_*) that also writes every activation
        # the backward edges read; the patch matrices the weight gradients multiply are then built beside the backward
        # chain.  False: layer by layer (im2col + GEMM convolutions), eleven launches.  Default: fused in f32, where a
        # replayed step takes 0.147-0.151 ms against 0.172; layered in bf16, where that launch is slower (0.175-0.181
        # against 0.164 ms: at batch 100 it is 25 workgroups walking twelve layers one after the other, and its bf16
        # form takes 30-47 us).
        if fused_forward is None:
            fused_forward = fused_backward or model.conv1.weight.dtype == "f32"
        self.fused_forward = fused_forward
        # fused_backward: the input-gradient chain (cross-entropy backward, three dense input gradients with their relu
        # backward, both pooling + relu backward passes, conv2's input gradient) is ONE launch, agh_lenet5_backward_*,
        # in place of nine; the weight gradients are the same GEMMs either way
        self.fused_backward = fused_backward
        # overlap: issue the weight gradients on the second stream beside the input-gradient chain.  Default: only for the
        # layer-by-layer backward pass; with the one-launch forms a step is six kernels, and the fork and join of a second
        # stream cost more (about 10 us) than the one launch they would hide
        if overlap is None:
            overlap = not fused_backward
        self._branch = branch if overlap else contextlib.nullcontext
        self.opt = optimizer if optimizer is not None else SGD()
        bs, dt = batch_size, model.conv1.weight.dtype
        self.dt = dt
        # `step` passes raw pointers of the input; the parameters are copied into one flat buffer below
        # (through standard-layout copies), so strided parameter views are fine, a strided x is not
        u = lambda *shape: Tensor.uninit(shape, dt)  # noqa: E731
        self.cols1, self.c1, self.p1 = u(bs * 576, 25), u(bs, 6, 24, 24), u(bs, 6, 12, 12)
        self.cols2, self.c2, self.p2 = u(bs * 64, 150), u(bs, 16, 8, 8), u(bs, 16, 4, 4)
        self.d1, self.a1, self.d2, self.a2, self.logits = u(bs, 128), u(bs, 128), u(bs, 84), u(bs, 84), u(bs, 10)
        self.g_logits, self.g_a2, self.g_d2 = u(bs, 10), u(bs, 84), u(bs, 84)
        self.g_a1, self.g_d1, self.g_f = u(bs, 128), u(bs, 128), u(bs, 256)
        # relu(conv) and the NCHW gradient of a convolution's output never exist: relu+pool and their backward
        # (which writes the [bs*h*w, c] matrix directly) are one launch each
        self.gm2 = u(bs * 64, 16)
        self.g_p1, self.gm1 = u(bs, 6, 12, 12), u(bs * 576, 6)
        # Parameters, gradients and velocities each live in ONE buffer (every tensor at a 128-byte aligned
        # offset, the gaps zero), so the element-wise update of all six parameters is a single launch.  The
        # model's layers are re-pointed at the views, so model and trainer share storage.
        m = model
        old = [m.conv1.weight, m.conv2.weight, m.dense1.weight, m.dense2.weight, m.dense3.weight, m.dense3.bias]
        offsets, total = [], 0
        for t in old:
            offsets.append(total)
            total += -(-len(t) // 64) * 64
        self._flat_len = total

        def views(flat):
            return [Tensor(flat.buffer, t.shape, _std_strides(t.shape), off, dt) for t, off in zip(old, offsets)]

        self._wflat, self._gflat = Tensor.zeros((total,), dt), Tensor.zeros((total,), dt)
        self.params, self.grads = views(self._wflat), views(self._gflat)
        for t, v in zip(old, self.params):
            src = t.as_standard_layout()
            check(lib.agh_memcpy_d2d(v._data_ptr(), src._data_ptr(), len(t) * _ITEMSIZE[dt]))
        check(lib.agh_sync())
        m.conv1.weight, m.conv2.weight, m.dense1.weight, m.dense2.weight, m.dense3.weight, m.dense3.bias = self.params
        if self.opt.momentum is not None:
            self._vflat = Tensor.zeros((total,), dt)
            self.velocities = views(self._vflat)
        else:
            self._vflat, self.velocities = None, [None] * 6
        # every parameter's optimizer state, as `SGD::init_state` builds it (optimizer.rs:358-381): named "SGD", empty
        # without momentum, else the velocity (a view of the shared buffer, so it is always current) marked as
        # following the parameter's device and type
        states = [OptimizerState("SGD", [] if v is None else [("velocity", v, True, True)]) for v in self.velocities]
        (m.conv1.weight_state, m.conv2.weight_state, m.dense1.weight_state, m.dense2.weight_state, m.dense3.weight_state,
         m.dense3.bias_state) = states
        host = C.c_void_p()
        check(lib.agh_host_alloc(C.byref(host), 4))
        self._loss_host = host
        self._graph = None

    def __del__(self):
        try:
            if getattr(self, "_graph", None):
                lib.agh_graph_destroy(self._graph)
            if getattr(self, "_loss_host", None):
                lib.agh_host_free(self._loss_host)
        except Exception:
            pass

    # raw launches on preallocated tensors
    def _fn(self, stem):
        return getattr(lib, f"{stem}_{self.dt}")

    def _conv_forward(self, x, weight, cols, y):
        bs, ic, ih, iw = x.shape
        oc, _, fh, fw = weight.shape
        oh, ow = ih - fh + 1, iw - fw + 1
        check(self._fn("agh_im2col_conv2")(x._data_ptr(), cols._ptr(), bs, ic, ih, iw, fh, fw, 0, 0, 1, 1, 1, 1))
        L, K = oh * ow, ic * fh * fw
        wm = weight.into_shape((oc, K))
        check(getattr(lib, f"agh_gemm_{self.dt}_batched")(
            bs, L, K, oc, 1.0, cols._ptr(), 0, K, 1, L * K, wm._ptr(), wm.offset, 1, K, 0,
            0.0, y._ptr(), 0, 1, L, oc * L, None, 0, 0, 0))

    def _relu_pool(self, x, y):
        """Relu then MaxPool2 2x2 (layer.rs:1253-1267, :1193-1216) in one launch; relu(x) is not kept."""
        bs, c, ih, iw = x.shape
        check(self._fn("agh_relu_max_pool2")(x._data_ptr(), y._ptr(), bs * c, ih, iw, 2, 2, 2, 2))

    def _pool_relu_backward(self, x, dy, out):
        """The backward of that pair from the relu's input x, written as the standard-layout [bs*h*w, c]
        matrix of the convolution backward (layer.rs:205-220, :1542-1565, autograd.rs:429-445): one launch for
        the pooling backward, the relu backward and the NHWC copy."""
        bs, c, ih, iw = x.shape
        check(self._fn("agh_max_pool2_relu_backward")(x._data_ptr(), dy._data_ptr(), out._ptr(), bs, c, ih, iw,
                                                      2, 2, 2, 2, 1))

    def _relu(self, x, y):
        check(self._fn("agh_relu")(x._data_ptr(), y._ptr(), len(x)))

    def _relu_backward(self, x, dy, dx):
        check(self._fn("agh_relu_backward")(x._data_ptr(), dy._data_ptr(), dx._ptr(), len(x)))

    def step(self, x, target):
        """x: [bs,1,28,28] tensor, target: device `Buffer` of bs u8 labels.  The loss lands in pinned
        host memory (`loss()` after a sync)."""
        bs = self.bs
        if not x.is_standard_layout() or x.shape != (bs, 1, 28, 28):
            raise AghError(-1, f"LeNet5Trainer.step: x must be a standard-layout [{bs},1,28,28] tensor")
        w1, w2, wd1, wd2, wd3, b3 = self.params
        dw1, dw2, dwd1, dwd2, dwd3, db3 = self.grads
        # forward
        f = self.p2.into_shape((bs, 256))
        if self.fused_forward:
            check(self._fn("agh_lenet5_forward_train")(
                x._data_ptr(), w1._data_ptr(), w2._data_ptr(), wd1._data_ptr(), wd2._data_ptr(), wd3._data_ptr(),
                b3._data_ptr(), self.c1._ptr(), self.p1._ptr(), self.c2._ptr(), self.p2._ptr(), self.d1._ptr(),
                self.a1._ptr(), self.d2._ptr(), self.a2._ptr(), self.logits._ptr(), bs))
            if not self.fused_backward:
                # the patch matrices feed only the weight gradients of the convolutions: built beside the backward chain
                # (the one-launch backward path forms those gradients without them)
                with self._branch():
                    check(self._fn("agh_im2col_conv2")(x._data_ptr(), self.cols1._ptr(), bs, 1, 28, 28, 5, 5, 0, 0, 1, 1, 1, 1))
                    check(self._fn("agh_im2col_conv2")(self.p1._ptr(), self.cols2._ptr(), bs, 6, 12, 12, 5, 5, 0, 0, 1, 1, 1, 1))
        else:
            self._conv_forward(x, w1, self.cols1, self.c1)
            self._relu_pool(self.c1, self.p1)
            self._conv_forward(self.p1, w2, self.cols2, self.c2)
            self._relu_pool(self.c2, self.p2)
            gemm(1.0, f, wd1, 0.0, self.d1)
            self._relu(self.d1, self.a1)
            gemm(1.0, self.a1, wd2, 0.0, self.d2)
            self._relu(self.d2, self.a2)
            gemm(1.0, self.a2, wd3, 0.0, self.logits, bias=b3)
        # backward.  The loss value and the weight gradients of the dense layers and of conv2 feed nothing
        # before the update:
        # with `overlap` they are issued together, once their operands exist, on the second stream, beside
        # the rest of the input-gradient chain (one fork and one join).
        def weight_grads():
            check(self._fn("agh_cross_entropy_loss")(self.logits._ptr(), target.ptr, bs, 10, self._loss_host))
            check(self._fn("agh_sum_axis0")(self.g_logits._ptr(), db3._data_ptr(), bs, 10))
            gemm(1.0, self.a2.t(), self.g_logits, 0.0, dwd3)
            gemm(1.0, self.a1.t(), self.g_d2, 0.0, dwd2)
            gemm(1.0, f.t(), self.g_d1, 0.0, dwd1)
            gemm(1.0, self.gm2.t(), self.cols2, 0.0, dw2.into_shape((16, 150)))

        if self.fused_backward:
            check(self._fn("agh_lenet5_backward")(
                self.logits._ptr(), target.ptr, 1.0, self.c1._ptr(), self.c2._ptr(), self.d1._ptr(), self.d2._ptr(),
                w2._data_ptr(), wd1._data_ptr(), wd2._data_ptr(), wd3._data_ptr(), self.g_logits._ptr(), self.g_d2._ptr(),
                self.g_d1._ptr(), self.gm2._ptr(), self.gm1._ptr(), bs))
            # everything below only waits for that launch: the dense layers' weight gradients, the bias gradient and the
            # loss are one launch on the second stream, the convolutions' weight gradients (formed without patch
            # matrices) two on the first
            with self._branch():
                check(self._fn("agh_lenet5_dense_weight_grads")(
                    self.a2._ptr(), self.a1._ptr(), f._data_ptr(), self.g_logits._ptr(), self.g_d2._ptr(), self.g_d1._ptr(),
                    dwd3._data_ptr(), dwd2._data_ptr(), dwd1._data_ptr(), db3._data_ptr(), self.logits._ptr(), target.ptr,
                    self._loss_host, bs))
            check(self._fn("agh_lenet5_conv_weight_grads")(x._data_ptr(), self.p1._ptr(), self.gm1._ptr(), self.gm2._ptr(),
                                                           dw1._data_ptr(), dw2._data_ptr(), bs))
            join()
        else:
            check(self._fn("agh_cross_entropy_backward")(self.logits._ptr(), target.ptr, 1.0, self.g_logits._ptr(), bs, 10))
            gemm(1.0, self.g_logits, wd3.t(), 0.0, self.g_a2)
            self._relu_backward(self.d2, self.g_a2, self.g_d2)
            gemm(1.0, self.g_d2, wd2.t(), 0.0, self.g_a1)
            self._relu_backward(self.d1, self.g_a1, self.g_d1)
            gemm(1.0, self.g_d1, wd1.t(), 0.0, self.g_f)
            self._pool_relu_backward(self.c2, self.g_f.into_shape((bs, 16, 4, 4)), self.gm2)
            with self._branch():
                weight_grads()
            # input gradient of conv2: dot with the weight matrix and col2im (layer.rs:976-988) in one launch
            check(self._fn("agh_conv2_backward_input")(self.gm2._ptr(), w2._data_ptr(), self.g_p1._ptr(), bs, 6, 8, 8, 16,
                                                       5, 5, 0, 0, 1, 1, 1, 1))
            self._pool_relu_backward(self.c1, self.g_p1, self.gm1)
            if self.fused_forward and self._branch is branch:
                join()  # the patch matrix of conv1 was built on the second stream
                gemm(1.0, self.gm1.t(), self.cols1, 0.0, dw1.into_shape((6, 25)))
            else:
                gemm(1.0, self.gm1.t(), self.cols1, 0.0, dw1.into_shape((6, 25)))
                join()
        # update: all parameters at once (element-wise, so one launch over the shared buffers)
        self.opt.update(self.lr, self._wflat, self._gflat, self._vflat)

    def loss(self):
        """The last step's loss; call after `agh_sync`."""
        return float(C.cast(self._loss_host, C.POINTER(C.c_float))[0])

    def capture(self, x, target):
        """Run one step eagerly (allocates the split-K workspace), then record a step into a graph.
        NOTE: both the eager step and the capture pass update the parameters."""
        self.step(x, target)
        check(lib.agh_sync())
        check(lib.agh_graph_begin())
        try:
            self.step(x, target)
        finally:
            g = C.c_void_p()
            check(lib.agh_graph_end(C.byref(g)))
        self._graph = g

    def replay(self):
        check(lib.agh_graph_launch(self._graph))
