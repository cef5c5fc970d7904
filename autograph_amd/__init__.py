"""MI355X-native device backend for autograph's dense-contraction hot path.

The package is a thin host layer over libautograph_hip.so; importing it fails loudly when
the library has not been built.
"""
from ._ffi import LIB_PATH, AghError, lib  # noqa: F401
from .layer import (  # noqa: F401
    Conv2,
    Dense,
    Flatten,
    LeNet5,
    LeNet5Trainer,
    MaxPool2,
    Relu,
    SGD,
    conv2_direct_forward,
    conv2_im2col_forward,
)
from .tensor import (  # noqa: F401
    BF16,
    F32,
    Buffer,
    Col2ImConv2Options,
    Device,
    Im2ColConv2Options,
    MaxPool2Options,
    Tensor,
    branch,
    gemm,
    join,
)
