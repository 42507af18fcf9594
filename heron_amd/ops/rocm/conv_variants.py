"""Convolutions the reference declares in other layouts or ranks, all served by the NHWC implicit-GEMM template.

The kernel reads an NHWC input and a KRSC filter; the adapter named in ``info['adapter']`` (``hostops.ADAPTERS``)
reorders the caller's operands once and reorders the result back.  The placeholders declared here are the kernel
operands, which is what the tuner measures.

  c1d_nwc   ops/cuda/conv1d.py:109-187   input (N,W,CI), filter (K,CI,CO)        -> conv2d with H = KH = 1
  c1d       ops/cuda/conv1d.py:11-107    input (N,CI,W), filter (CO,CI,KW)       -> the same after NCW -> NWC
  c2d_nchw  ops/cuda/conv2d.py:9-135     input (N,CI,H,W), filter (CO,CI,KH,KW); CI is zero-padded to a whole 16-byte
                                         chunk (the reference pads the filter window instead for CI = 3, conv2d.py:31-52)
  dil       ops/cuda/dil.py:8-105        NHWC input, HWIO filter (KH,KW,CI,CO), dilation >= 1
  c3d_ndhwc ops/cuda/conv3d.py:117-234   input (N,D,H,W,CI), filter (KD,KH,KW,CI,CO): the depth taps are unfolded into
                                         the channel axis (KD*CI channels, N*DO images), height and width stay implicit
  c3d       ops/cuda/conv3d.py:10-115    input (N,CI,D,H,W), filter (CO,CI,KD,KH,KW) -> the same after NCDHW -> NDHWC
  t2d       ops/cuda/conv2d_transposed.py:59-171  input (N,CI,H,W), filter (CO,CI,KH,KW): zero-expand by the stride,
                                         pad by dilated_K-1-padding (+outpadding after), then a stride-1 correlation
                                         with the filter as stored.  (The reference multiplies the output position by
                                         the stride once more when it indexes the expanded input,
                                         conv2d_transposed.py:103-104, which reads past the padded tensor for stride > 1;
                                         the well-defined stride-1 reading of that expression is what is built.)
"""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info
from .conv2d import conv_out_size, pair


def _chunk_elems(kind):
    return 8 if kind == "f16" else 16


def _declare(ctx, kind, N, H, W, CI, CO, KH, KW, stride, pad, dil, adapter, reference_args, extra=None):
    """Kernel-side conv2d NHWC x KRSC declaration with (h, w) stride/pad/dil pairs."""
    (sh, sw), (ph, pw), (dh, dw) = pair(stride), pair(pad), pair(dil)
    HO, WO = conv_out_size(H, KH, sh, ph, dh), conv_out_size(W, KW, sw, pw, dw)
    if HO <= 0 or WO <= 0:
        raise ValueError("empty convolution output")
    a_dt, b_dt, o_dt = ("float16", "float16", "float16") if kind == "f16" else ("uint8", "int8", "int32")
    Input = placeholder((N, H, W, CI), "input", a_dt)
    Filter = placeholder((CO, KH, KW, CI), "filter", b_dt)
    out = compute((N, HO, WO, CO), "out", o_dt, [Input, Filter], tag="conv2d_nhwc_mfma")
    conv = dict(w_format=None, N=N, H=H, W=W, CI=CI, CO=CO, KH=KH, KW=KW, stride=sh, pad=ph, dil=dh,
                stride_w=sw, pad_w=pw, dil_w=dw, HO=HO, WO=WO)
    info = {'conv': conv, 'adapter': adapter, 'reference_args': reference_args}
    info.update(extra or {})
    ctx.set_info(mfma_info(kind, out.op.name, Input.name, Filter.name,
                           dict(batch=1, M=N * HO * WO, N=CO, K=KH * KW * CI), 'conv2d_nhwc', info))
    ctx.set_axis_map({
        'input.lds': ['s_0', 's_1', 's_2', 'r_0', 'r_1', 'r_2'],
        'filter.lds': ['s_3', 'r_0', 'r_1', 'r_2'],
        'out.mfma.accumulator': ['s_0', 's_1', 's_2', 's_3'],
    })
    return [out]


def _ci_padded(CI, kind):
    q = _chunk_elems(kind)
    return (CI + q - 1) // q * q


def heron_conv1d_nwc(ctx, N, W, CI, CO, K, stride, padding, dilation, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    ref = dict(input=(N, W, CI), filter=(K, CI, CO))
    return _declare(ctx, kind, N, 1, W, _ci_padded(CI, kind), CO, 1, K, (1, stride), (0, padding), (1, dilation),
                    'c1d_nwc', ref, {'ci': CI})


def heron_conv1d_ncw(ctx, N, W, CI, CO, KW, stride, padding, dilation, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    ref = dict(input=(N, CI, W), filter=(CO, CI, KW))
    return _declare(ctx, kind, N, 1, W, _ci_padded(CI, kind), CO, 1, KW, (1, stride), (0, padding), (1, dilation),
                    'c1d_ncw', ref, {'ci': CI})


def heron_conv2d_nchw(ctx, N, H, W, CI, CO, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    ref = dict(input=(N, CI, H, W), filter=(CO, CI, KH, KW))
    return _declare(ctx, kind, N, H, W, _ci_padded(CI, kind), CO, KH, KW, stride, padding, dilation, 'c2d_nchw', ref,
                    {'ci': CI})


def heron_dil_nhwc(ctx, N, H, W, CI, CO, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    ref = dict(input=(N, H, W, CI), filter=(KH, KW, CI, CO))
    return _declare(ctx, kind, N, H, W, _ci_padded(CI, kind), CO, KH, KW, stride, padding, dilation, 'c2d_hwio', ref,
                    {'ci': CI})


def _triple(v):
    return (int(v),) * 3 if isinstance(v, int) else tuple(int(x) for x in v)


def _conv3d(ctx, layout, N, D, H, W, CI, CO, KD, KH, KW, stride, padding, dilation, in_dtype):
    kind = element_kind(in_dtype)
    (sd, sh, sw), (pd, ph, pw), (dd, dh, dw) = _triple(stride), _triple(padding), _triple(dilation)
    DO = conv_out_size(D, KD, sd, pd, dd)
    if DO <= 0:
        raise ValueError("empty convolution output")
    cip = _ci_padded(CI, kind)
    ref = dict(input=(N, D, H, W, CI), filter=(KD, KH, KW, CI, CO)) if layout == 'ndhwc' else \
        dict(input=(N, CI, D, H, W), filter=(CO, CI, KD, KH, KW))
    extra = {'ci': CI, 'depth': dict(D=D, KD=KD, DO=DO, stride=sd, pad=pd, dil=dd, N=N)}
    return _declare(ctx, kind, N * DO, H, W, KD * cip, CO, KH, KW, (sh, sw), (ph, pw), (dh, dw), 'c3d_' + layout, ref, extra)


def heron_conv3d_ndhwc(ctx, N, D, H, W, CI, CO, KD, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    return _conv3d(ctx, 'ndhwc', N, D, H, W, CI, CO, KD, KH, KW, stride, padding, dilation, in_dtype)


def heron_conv3d_ncdhw(ctx, N, D, H, W, CI, CO, KD, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    return _conv3d(ctx, 'ncdhw', N, D, H, W, CI, CO, KD, KH, KW, stride, padding, dilation, in_dtype)


def heron_conv2d_nchw_transposed(ctx, N, H, W, CI, CO, KH, KW, stride, padding, dilation, outpadding, in_dtype,
                                 out_dtype):
    assert isinstance(stride, int) and isinstance(padding, int) and isinstance(dilation, int)
    kind = element_kind(in_dtype)
    dkh, dkw = (KH - 1) * dilation + 1, (KW - 1) * dilation + 1
    if dkh - 1 - padding < 0 or dkw - 1 - padding < 0:
        raise ValueError("padding larger than the dilated filter")
    # the expanded and padded tensor the kernel convolves (conv2d_transposed.py:83-94)
    HE = (H - 1) * stride + 1 + 2 * (dkh - 1 - padding) + outpadding
    WE = (W - 1) * stride + 1 + 2 * (dkw - 1 - padding) + outpadding
    ref = dict(input=(N, CI, H, W), filter=(CO, CI, KH, KW))
    extra = {'ci': CI, 'transposed': dict(stride=stride, pad=padding, dil=dilation, outpad=outpadding, H=H, W=W)}
    return _declare(ctx, kind, N, HE, WE, _ci_padded(CI, kind), CO, KH, KW, 1, 0, dilation, 't2d_nchw', ref, extra)
