"""MFMA operator set for gfx950: same registry and signatures as ops/cuda and ops/x86 of the reference.

``getOpFromName`` (ops/cuda/__init__.py:15-32, ops/x86/__init__.py:11-23) maps the ``cases`` entry of
a config JSON to an operator definition ``opfunc(ctx, *shape, in_dtype, out_dtype) -> [out]``.
"""
from .dense import heron_dense
from .batch_matmul import heron_batch_matmul
from .conv2d import heron_conv2d_nhwc
from .conv_variants import (heron_conv1d_ncw, heron_conv1d_nwc, heron_conv2d_nchw, heron_conv2d_nchw_transposed,
                            heron_conv3d_ncdhw, heron_conv3d_ndhwc, heron_dil_nhwc)
from .reductions import heron_depthwise_conv2d, heron_gemv, heron_mean, heron_scan, heron_var


class _tolerates_w_format:
    """The x86 operator set passes the name of its blocked weight layout ("OwI64o4i", "OdhwI64o4i", "OIhw4i16o4i", ...)
    as the last shape argument (ops/x86/conv1d_int8.py, conv3d_int8.py, dil.py, t2d.py; cases of tests/figure8/configs).
    The MFMA operators take the filter in the layout their docstring names, so the entry is accepted and dropped.
    (A class rather than a closure: tasks travel to forked sampler processes and back through pickles.)"""

    def __init__(self, opfunc):
        self.opfunc = opfunc
        self.__name__ = opfunc.__name__
        self.__doc__ = opfunc.__doc__

    def __call__(self, ctx, *args):
        *shape, in_dtype, out_dtype = args
        if shape and isinstance(shape[-1], str):
            shape = shape[:-1]
        return self.opfunc(ctx, *shape, in_dtype, out_dtype)


def getOpFromName(name):
    opmap = {
        "gemm": heron_dense,
        "bmm": heron_batch_matmul,
        "c2d": heron_conv2d_nhwc,                 # NHWC, as ops/x86 and the benchmark configs; NCHW is "c2d_nchw"
        "c2d_nhwc": heron_conv2d_nhwc,
        "c2d_nchw": heron_conv2d_nchw,
        "gemv": heron_gemv,
        "scan": heron_scan,
        "mean": heron_mean,
        "var": heron_var,
        "c1d": heron_conv1d_ncw,
        "c1d_nwc": heron_conv1d_nwc,
        "c3d": heron_conv3d_ncdhw,
        "c3d_ndhwc": heron_conv3d_ndhwc,
        "dil": heron_dil_nhwc,
        "t2d": heron_conv2d_nchw_transposed,
        "dep": heron_depthwise_conv2d,
    }
    if name in ("c1d", "c1d_nwc", "c3d", "c3d_ndhwc", "dil", "t2d", "c2d_nchw"):
        return _tolerates_w_format(opmap[name])
    return opmap[name]
