"""Operators the reference expresses as a GEMM against a constant or padded right-hand side.

Each one follows the declaration of its TensorCore counterpart: the operands the user passes are turned
into the (M,K) x (N,K) form by an injective pre-stage, and the product runs on the matrix units.  Here the
pre-stage is the operand adapter named in ``info['adapter']`` (``hostops.ADAPTERS``) and the product is the
MFMA GEMM template; the placeholders below are the *kernel* operands, which is what the tuner measures.

  gemv   ops/cuda/gemv.py:4-65     out (M,8) = A (M,K) x pad8(B (1,K)); column 0 holds A.b
  scan   ops/cuda/scan.py:4-59     out (M,N) = A (M,K) x T (N,K), T[n,k] = 1 if n > k else 0: exclusive prefix sums
  mean   ops/cuda/mean.py:4-66     out (C,8) = A (C,N*H*W) x B (8,N*H*W), B[0,:] = 1/(N*H*W): per-channel mean of NCHW
  var    ops/cuda/var.py:4-75      the same product applied to (In - Mean)**2
  dep    ops/cuda/dep.py:9-123     depthwise 3x3 conv as one small product per channel: batch = C, A (C, N*HO*WO, 16) the
                                   3x3 windows padded to 4x4 taps, B (C, 8, 16) the channel's K/C filters padded to 8 rows,
                                   out (N, C, 8, HO, WO)
"""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info

PAD_N = 8          # the reference pads the single right-hand-side row to 8 rows (gemv.py:6,11)


def _declare(ctx, kind, M, N, K, adapter, reference_args, extra=None):
    a_dt, b_dt, o_dt = ("float16", "float16", "float16") if kind == "f16" else ("uint8", "int8", "int32")
    A = placeholder((M, K), "A", a_dt)
    B = placeholder((N, K), "B", b_dt)
    out = compute((M, N), "dense", o_dt, [A, B], tag="matmul")
    info = {'adapter': adapter, 'reference_args': reference_args}
    info.update(extra or {})
    ctx.set_info(mfma_info(kind, out.op.name, A.name, B.name, dict(batch=1, M=M, N=N, K=K), 'gemm', info))
    ctx.set_axis_map({'A.lds': ['s_0', 'r_0'], 'B.lds': ['s_1', 'r_0'], 'dense.mfma.accumulator': ['s_0', 's_1']})
    return [out]


def _k_padded(K, kind):
    q = 8 if kind == "f16" else 16            # K rows are moved in 16-byte chunks
    return (K + q - 1) // q * q


def heron_gemv(ctx, M, K, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    return _declare(ctx, kind, M, PAD_N, _k_padded(K, kind), 'gemv', dict(A=(M, K), B=(1, K), out=(M, PAD_N)))


def heron_scan(ctx, M, N, K, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    return _declare(ctx, kind, M, N, _k_padded(K, kind), 'scan', dict(A=(M, K), out=(M, N)))


def heron_mean(ctx, N, C, H, W, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    if kind != "f16":
        raise ValueError("mean multiplies by 1/(N*H*W): floating point only")
    return _declare(ctx, kind, C, PAD_N, _k_padded(N * H * W, kind), 'mean', dict(In=(N, C, H, W), out=(C, PAD_N)))


def heron_var(ctx, N, C, H, W, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    if kind != "f16":
        raise ValueError("var multiplies by 1/(N*H*W): floating point only")
    return _declare(ctx, kind, C, PAD_N, _k_padded(N * H * W, kind), 'var',
                    dict(In=(N, C, H, W), Mean=(N, C, H, W), out=(C, PAD_N)))


def heron_depthwise_conv2d(ctx, N, H, W, C, K, KH, KW, stride, padding, dilation, in_dtype, out_dtype):
    """Depthwise conv of an NCHW input with K = multiplier * C filters (K, 3, 3), declared as the reference declares it
    (dep.py:9-123): a batched product over channels with M = N*HO*WO pixels, the 3x3 window zero-padded to 4x4 = 16
    taps as K, and the channel's filters zero-padded to 8 rows as N."""
    assert isinstance(stride, int) and dilation == 1 and K % C == 0 and KH == 3 and KW == 3
    kind = element_kind(in_dtype)
    HO = (H - KH + 2 * padding) // stride + 1
    WO = (W - KW + 2 * padding) // stride + 1
    mult = K // C
    NP = (mult + 7) // 8 * 8
    a_dt, b_dt, o_dt = ("float16", "float16", "float16") if kind == "f16" else ("uint8", "int8", "int32")
    A = placeholder((C, N * HO * WO, 16), "A", a_dt)
    B = placeholder((C, NP, 16), "B", b_dt)
    out = compute((C, N * HO * WO, NP), "C", o_dt, [A, B], tag="batch_matmul")
    info = {'adapter': 'dep', 'reference_args': dict(input=(N, C, H, W), filter=(K, KH, KW), out=(N, C, NP, HO, WO)),
            'dep': dict(N=N, C=C, H=H, W=W, K=K, stride=stride, pad=padding, HO=HO, WO=WO, mult=mult, NP=NP)}
    ctx.set_info(mfma_info(kind, out.op.name, A.name, B.name, dict(batch=C, M=N * HO * WO, N=NP, K=16), 'gemm', info))
    ctx.set_axis_map({'A.lds': ['s_1', 'r_0'], 'B.lds': ['s_2', 'r_0'], 'C.mfma.accumulator': ['s_0', 's_1', 's_2']})
    return [out]
