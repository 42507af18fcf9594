"""conv2d NHWC as implicit GEMM on MFMA (fp16, and the quantized uint8 x int8 -> int32 form).

Out[n,y,x,f] = sum_{ry,rx,rc} Pad(In)[n, y*s + ry*d, x*s + rx*d, rc] * W[f,ry,rx,rc]
(ops/cuda/conv2d.py:137-232).  The filter is taken in KRSC order (CO,KH,KW,CI) - the reference
stores HWIO (KH,KW,CI,CO) - so that, in GEMM terms, B is (N,K) with K = (ry,rx,rc) contiguous,
the same operand form as dense.  GEMM view: M = N*HO*WO, N = CO, K = KH*KW*CI; the im2col
addresses are generated inside the kernel and padding taps are read as zeros.

Quantized form (ops/x86/conv2d_int8.py:31-109): uint8 NHWC input, int8 filter, int32 output.  The
reference signature carries a ``w_format`` ("OhwI64o4i" | "OhwI48o4i" | "OhwI32o4i") naming its blocked
filter (CO/b,KH,KW,CI/4,b,4) and yields a 5-d output (N,HO,WO,CO/b,b); the kernel takes the filter in
KRSC order and writes (N,HO,WO,CO), which is that output seen flat.  ``w_format`` is accepted in the
same position and recorded in the operator info so that callers holding blocked weights know to
reorder them once (``hostops.unpack_filter_blocked``).
"""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info


def pair(v):
    """int or (height, width) pair, as the reference's operators accept (ops/cuda/conv2d.py:143-153)."""
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def conv_out_size(size, k, stride, pad, dil):
    return (size - ((k - 1) * dil + 1) + 2 * pad) // stride + 1


W_FORMATS = ("OhwI64o4i", "OhwI48o4i", "OhwI32o4i")


def heron_conv2d_nhwc(ctx, N, H, W, CI, CO, KH, KW, stride, padding, dilation, *dtypes):
    """``dtypes`` is (in_dtype, out_dtype) as in ops/cuda/conv2d.py:137-141, or (w_format, in_dtype, out_dtype)
    as in ops/x86/conv2d_int8.py:31-35."""
    (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(padding), pair(dilation)
    w_format = None
    if len(dtypes) == 3:
        w_format, in_dtype, out_dtype = dtypes
        assert w_format in W_FORMATS
        # (the reference floors CO to whole filter blocks, conv2d_int8.py:50,75; the KRSC filter has no blocks, so
        # every output channel is computed)
    else:
        in_dtype, out_dtype = dtypes
    kind = element_kind(in_dtype)
    if w_format is not None and kind != "u8s8":
        raise ValueError("w_format belongs to the quantized operator")
    chunk = 8 if kind == "f16" else 16
    extra = {}
    if CI % chunk:
        # fewer channels than a whole 16-byte chunk (the 3-channel stem of the vision networks): the kernel runs on
        # zero-padded channels, the 'c2d_krsc' adapter pads activation and filter, the result needs no reorder
        extra = {'adapter': 'c2d_krsc', 'reference_args': dict(input=(N, H, W, CI), filter=(CO, KH, KW, CI)), 'ci': CI}
        CI = (CI + chunk - 1) // chunk * chunk
    HO = conv_out_size(H, KH, sh, ph, dh)
    WO = conv_out_size(W, KW, sw, pw, dw)
    a_dt, b_dt, o_dt = ("float16", "float16", "float16") if kind == "f16" else ("uint8", "int8", "int32")
    Input = placeholder((N, H, W, CI), "input", a_dt)
    Filter = placeholder((CO, KH, KW, CI), "filter", b_dt)
    out = compute((N, HO, WO, CO), "out", o_dt, [Input, Filter], tag="conv2d_nhwc_mfma")
    conv = dict(w_format=w_format, N=N, H=H, W=W, CI=CI, CO=CO, KH=KH, KW=KW, stride=sh, pad=ph, dil=dh, stride_w=sw, pad_w=pw, dil_w=dw,
                HO=HO, WO=WO)
    ctx.set_info(mfma_info(kind, out.op.name, Input.name, Filter.name,
                           dict(batch=1, M=N * HO * WO, N=CO, K=KH * KW * CI), 'conv2d_nhwc', dict(extra, conv=conv)))
    ctx.set_axis_map({
        'input.lds': ['s_0', 's_1', 's_2', 'r_0', 'r_1', 'r_2'],
        'filter.lds': ['s_3', 'r_0', 'r_1', 'r_2'],
        'out.mfma.accumulator': ['s_0', 's_1', 's_2', 's_3'],
    })
    return [out]
