"""GEMM operator: C[i,j] = sum_k A[i,k] * B[j,k].

fp16 operands follow ops/cuda/dense.py:4-54 (A (M,K) row-major, B (N,K) i.e. column-major), with the
accumulation in fp32 and one rounding to fp16 on store.  Quantized operands follow
ops/x86/dense.py:6-32: A uint8, B int8, int32 accumulate and output.
"""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info


def heron_dense(ctx, M, K, N, in_dtype, out_dtype):
    kind = element_kind(in_dtype)
    if kind == "f16":
        A = placeholder((M, K), "A", "float16")
        B = placeholder((N, K), "B", "float16")
        out = compute((M, N), "dense", "float16", [A, B], tag="batch_matmul")
    else:
        A = placeholder((M, K), "A", "uint8")
        B = placeholder((N, K), "B", "int8")
        out = compute((M, N), "dense", "int32", [A, B], tag="batch_matmul")
    ctx.set_info(mfma_info(kind, out.op.name, A.name, B.name, dict(batch=1, M=M, N=N, K=K), 'gemm'))
    ctx.set_axis_map({
        'A.lds': ['s_0', 'r_0'],
        'B.lds': ['s_1', 'r_0'],
        'dense.mfma.accumulator': ['s_0', 's_1'],
    })
    return [out]
