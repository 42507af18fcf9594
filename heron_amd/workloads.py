"""Seeded synthetic inputs for the benchmark configurations, and their algorithmic work/bytes.

Distributions: uint8 uniform[0,255] x int8 uniform[-128,127] for the quantized GEMMs; fp16
N(0,1)*0.1 for the dense GEMM; ReLU'd N(0,1) activations and N(0,0.05) KRSC weights for the
conv; N(0,1) Q/K/V and row-softmax P for the attention batch_matmuls.  numpy only.
"""
import numpy as np


def gemm_u8s8_inputs(M, K, N, seed=0):
    """A (M,K) uint8, B (N,K) int8 - operand layout of ops/x86/dense.py:7-11 in the reference."""
    rng = np.random.default_rng(seed)
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    B = rng.integers(-128, 128, size=(N, K), dtype=np.int8)
    return A, B


def gemm_f16_inputs(M, K, N, seed=1, scale=0.1):
    """A (M,K), B (N,K) fp16 ~ N(0,1)*scale - layout of ops/cuda/dense.py:5-9."""
    rng = np.random.default_rng(seed)
    A = (rng.standard_normal((M, K), dtype=np.float32) * scale).astype(np.float16)
    B = (rng.standard_normal((N, K), dtype=np.float32) * scale).astype(np.float16)
    return A, B


def bmm_qk_inputs(batch, M, K, N, seed=4):
    """Q (b,M,K), K (b,N,K) fp16 ~ N(0,1): the Q.K^T product of one attention layer."""
    rng = np.random.default_rng(seed)
    Q = rng.standard_normal((batch, M, K), dtype=np.float32).astype(np.float16)
    Kt = rng.standard_normal((batch, N, K), dtype=np.float32).astype(np.float16)
    return Q, Kt


def bmm_pv_inputs(batch, M, K, N, seed=5):
    """P (b,M,K) row-softmax of N(0,1), V^T (b,N,K) ~ N(0,1): the P.V product, V stored transposed."""
    rng = np.random.default_rng(seed)
    S = rng.standard_normal((batch, M, K), dtype=np.float32)
    S = np.exp(S - S.max(axis=-1, keepdims=True))
    P = (S / S.sum(axis=-1, keepdims=True)).astype(np.float16)
    Vt = rng.standard_normal((batch, N, K), dtype=np.float32).astype(np.float16)
    return P, Vt


def conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=3):
    """Input NHWC fp16 = relu(N(0,1)) (about half zeros), filter KRSC (CO,KH,KW,CI) fp16 ~ N(0,0.05)."""
    rng = np.random.default_rng(seed)
    X = np.maximum(rng.standard_normal((N, H, W, CI), dtype=np.float32), 0).astype(np.float16)
    Wt = (rng.standard_normal((CO, KH, KW, CI), dtype=np.float32) * 0.05).astype(np.float16)
    return X, Wt


def conv2d_u8s8_inputs(N, H, W, CI, CO, KH, KW, seed=6):
    """uint8 NHWC activations and int8 KRSC weights over their full ranges (ops/x86/conv2d_int8.py:51-52)."""
    rng = np.random.default_rng(seed)
    X = rng.integers(0, 256, (N, H, W, CI), dtype=np.uint8)
    Wt = rng.integers(-128, 128, (CO, KH, KW, CI), dtype=np.int8)
    return X, Wt


def conv_out_hw(H, W, KH, KW, stride, pad, dil):
    """Output size formula of ops/cuda/conv2d.py:168-175."""
    ho = (H - ((KH - 1) * dil + 1) + 2 * pad) // stride + 1
    wo = (W - ((KW - 1) * dil + 1) + 2 * pad) // stride + 1
    return ho, wo


def gemm_work(M, N, K, in_bytes, out_bytes, batch=1):
    """(operations, algorithmic bytes): 2MNK and each operand read once + the result written once."""
    return 2 * batch * M * N * K, batch * ((M * K + N * K) * in_bytes + M * N * out_bytes)


def conv_work(N, H, W, CI, CO, KH, KW, stride, pad, dil, in_bytes=2, out_bytes=2):
    ho, wo = conv_out_hw(H, W, KH, KW, stride, pad, dil)
    ops = 2 * N * ho * wo * CO * KH * KW * CI      # padding taps counted
    byts = (N * H * W * CI + CO * KH * KW * CI) * in_bytes + N * ho * wo * CO * out_bytes
    return ops, byts


# published dense peaks of MI355X used as roofline denominators
PEAK_FP16_TFLOPS = 2500.0
PEAK_INT8_TOPS = 5000.0
PEAK_HBM_GBS = 8000.0
