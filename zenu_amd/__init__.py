"""zenu_amd -- MI355X (gfx950) device tensor-kernel layer for ZeNu.

`zenu_amd.lib/libzenu_hip.so` is the product: hand-written HIP kernels behind the C ABI of
include/zenu_hip.h.  This package is the thin host-side mirror of zenu-matrix's Matrix /
zenu-optimizer's optimizers used by the tests and the benchmark.
"""
from ._lib import ZenuHipError, lib, LIB_PATH  # noqa: F401
from .matrix import (Matrix, sum_to, larger_shape, set_stream, get_stream, synchronize, default_stride,  # noqa: F401
                     softmax_backward, cross_entropy, cross_entropy_backward, cross_entropy_backward_bias_grad,
                     conv2d_bias_add,
                     conv2d_bias_bkwd, stack, split)
from .optim import SGD, Adam, AdamW  # noqa: F401
from . import checkpoint  # noqa: F401
