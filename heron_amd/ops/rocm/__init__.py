"""MFMA operator set for gfx950: same registry and signatures as ops/cuda and ops/x86 of the reference.

``getOpFromName`` (ops/cuda/__init__.py:15-32, ops/x86/__init__.py:11-23) maps the ``cases`` entry of
a config JSON to an operator definition ``opfunc(ctx, *shape, in_dtype, out_dtype) -> [out]``.
"""
from .dense import heron_dense
from .batch_matmul import heron_batch_matmul
from .conv2d import heron_conv2d_nhwc


def getOpFromName(name):
    opmap = {
        "gemm": heron_dense,
        "bmm": heron_batch_matmul,
        "c2d": heron_conv2d_nhwc,
        "c2d_nhwc": heron_conv2d_nhwc,
    }
    return opmap[name]
