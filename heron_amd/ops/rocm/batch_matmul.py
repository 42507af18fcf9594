"""batch_matmul operator: C[b,i,j] = sum_k A[b,i,k] * B[b,j,k]  (ops/cuda/batch_matmul.py:5-56,
ops/x86/batch_matmul.py:6-34); the batch index becomes an outer dimension of the tile grid."""
from ..tensor import compute, placeholder
from .common import element_kind, mfma_info


def heron_batch_matmul(ctx, batch, M, K, N, in_dtype, out_dtype):
    assert batch > 1
    kind = element_kind(in_dtype)
    a_dt, b_dt, o_dt = ("float16", "float16", "float16") if kind == "f16" else ("uint8", "int8", "int32")
    A = placeholder((batch, M, K), "A", a_dt)
    B = placeholder((batch, N, K), "B", b_dt)
    out = compute((batch, M, N), "batch_matmul", o_dt, [A, B], tag="batch_matmul")
    ctx.set_info(mfma_info(kind, out.op.name, A.name, B.name, dict(batch=batch, M=M, N=N, K=K), 'gemm'))
    ctx.set_axis_map({
        'A.lds': ['s_1', 'r_0'],
        'B.lds': ['s_2', 'r_0'],
        'batch_matmul.mfma.accumulator': ['s_0', 's_1', 's_2'],
    })
    return [out]
