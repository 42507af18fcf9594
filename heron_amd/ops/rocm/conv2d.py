"""conv2d NHWC as implicit GEMM on MFMA.

Out[n,y,x,f] = sum_{ry,rx,rc} Pad(In)[n, y*s + ry*d, x*s + rx*d, rc] * W[f,ry,rx,rc]
(ops/cuda/conv2d.py:137-232).  The filter is taken in KRSC order (CO,KH,KW,CI) - the reference
stores HWIO (KH,KW,CI,CO) - so that, in GEMM terms, B is (N,K) with K = (ry,rx,rc) contiguous,
the same operand form as dense.  GEMM view: M = N*HO*WO, N = CO, K = KH*KW*CI; the im2col
addresses are generated inside the kernel and padding taps are read as zeros.
"""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info


def conv_out_size(size, k, stride, pad, dil):
    return (size - ((k - 1) * dil + 1) + 2 * pad) // stride + 1


def heron_conv2d_nhwc(ctx, N, H, W, CI, CO, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    assert isinstance(stride, int) and isinstance(padding, int) and isinstance(dilation, int), \
        "square stride/padding/dilation"
    kind = element_kind(in_dtype)
    if kind != "f16":
        raise ValueError("conv2d_nhwc on MFMA is fp16 only")
    if CI % 8:
        raise ValueError("CI must be a multiple of 8 (16-byte channel chunks)")
    HO = conv_out_size(H, KH, stride, padding, dilation)
    WO = conv_out_size(W, KW, stride, padding, dilation)
    Input = placeholder((N, H, W, CI), "input", "float16")
    Filter = placeholder((CO, KH, KW, CI), "filter", "float16")
    out = compute((N, HO, WO, CO), "out", "float16", [Input, Filter], tag="conv2d_nhwc_mfma")
    conv = dict(N=N, H=H, W=W, CI=CI, CO=CO, KH=KH, KW=KW, stride=stride, pad=padding, dil=dilation, HO=HO, WO=WO)
    ctx.set_info(mfma_info(kind, out.op.name, Input.name, Filter.name,
                           dict(batch=1, M=N * HO * WO, N=CO, K=KH * KW * CI), 'conv2d_nhwc', {'conv': conv}))
    ctx.set_axis_map({
        'input.lds': ['s_0', 's_1', 's_2', 'r_0', 'r_1', 'r_2'],
        'filter.lds': ['s_3', 'r_0', 'r_1', 'r_2'],
        'out.mfma.accumulator': ['s_0', 's_1', 's_2', 's_3'],
    })
    return [out]
