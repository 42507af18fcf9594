"""Python face of the CPU oracle (test infrastructure, never on the product path).

Two independent restatements of each operator live here:

* the C functions of ``heron_oracle.c`` (loaded with ctypes from ``liboracle.so``), and
* closed forms in numpy (int64 matmul for the integer path, float64 einsum for the
  floating point ones).

``tests/test_oracle.py`` pins them against each other, against brute force loops, torch's CPU
``conv2d`` and extreme-value closed forms.  Reference lines each one follows are cited in
``heron_oracle.c``.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


def build(force=False):
    """Compile ``liboracle.so`` with the Makefile next to this file."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_num_threads.restype = ctypes.c_int
        L.orc_has_vnni.restype = ctypes.c_int
        L.orc_gemm_u8s8s32_scalar.argtypes = [_p, _p, _p, _i64, _i64, _i64]
        L.orc_bmm_u8s8s32_scalar.argtypes = [_p, _p, _p, _i64, _i64, _i64, _i64]
        L.orc_gemm_u8s8s32_dlboost.argtypes = [_p, _p, _p, _i64, _i64, _i64]
        L.orc_gemm_u8s8s32_dlboost.restype = ctypes.c_int
        L.orc_pack_b.argtypes = [_p, _i64, _i64]
        L.orc_pack_b.restype = _p
        L.orc_free_b.argtypes = [_p]
        L.orc_gemm_u8s8s32_packed.argtypes = [_p, _p, _p, _i64, _i64, _i64]
        L.orc_gemm_u8s8s32_packed.restype = ctypes.c_int
        L.orc_gemm_f32.argtypes = [_p, _p, _p, _i64, _i64, _i64]
        L.orc_bmm_f32.argtypes = [_p, _p, _p, _i64, _i64, _i64, _i64]
        L.orc_conv2d_nhwc_f32.argtypes = [_p, _p, _p] + [_i64] * 10
        L.orc_conv2d_nhwc_u8s8s32.argtypes = [_p, _p, _p] + [_i64] * 10
        L.orc_conv2d_nhwc_u8s8s32_blocked.argtypes = [_p, _p, _p] + [_i64] * 11
        L.orc_conv2d_nhwc_u8s8s32_blocked.restype = ctypes.c_int
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data_as(_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def num_threads():
    return int(lib().orc_num_threads())


def has_vnni():
    return bool(lib().orc_has_vnni())


# ---------------------------------------------------------------- integer path
def gemm_u8s8s32_scalar(A, B):
    """C triple loop.  A (M,K) uint8, B (N,K) int8 -> (M,N) int32."""
    A = _c(A, np.uint8); B = _c(B, np.int8)
    M, K = A.shape; N = B.shape[0]
    assert B.shape[1] == K
    C = np.empty((M, N), np.int32)
    lib().orc_gemm_u8s8s32_scalar(_ptr(A), _ptr(B), _ptr(C), M, N, K)
    return C


def gemm_u8s8s32_dlboost(A, B, return_path=False):
    """DL Boost-structured path (16x4 ``vpdpbusd`` micro-kernel, OpenMP outer tiles)."""
    A = _c(A, np.uint8); B = _c(B, np.int8)
    M, K = A.shape; N = B.shape[0]
    assert B.shape[1] == K
    C = np.empty((M, N), np.int32)
    path = lib().orc_gemm_u8s8s32_dlboost(_ptr(A), _ptr(B), _ptr(C), M, N, K)
    return (C, path) if return_path else C


class PackedB:
    """Weights re-packed once to the 16x4 block layout the micro-kernel loads."""

    def __init__(self, B):
        B = _c(B, np.int8)
        self.N, self.K = B.shape
        self.handle = lib().orc_pack_b(_ptr(B), self.N, self.K)
        if not self.handle:
            raise RuntimeError("orc_pack_b: no AVX512-VNNI or N%32 / K%4 != 0")

    def matmul(self, A, out=None):
        A = _c(A, np.uint8)
        M = A.shape[0]
        C = out if out is not None else np.empty((M, self.N), np.int32)
        rc = lib().orc_gemm_u8s8s32_packed(_ptr(A), self.handle, _ptr(C), M, self.N, self.K)
        assert rc == 0
        return C

    def __del__(self):
        if getattr(self, "handle", None):
            lib().orc_free_b(self.handle)
            self.handle = None


def bmm_u8s8s32_scalar(A, B):
    A = _c(A, np.uint8); B = _c(B, np.int8)
    b, M, K = A.shape; N = B.shape[1]
    C = np.empty((b, M, N), np.int32)
    lib().orc_bmm_u8s8s32_scalar(_ptr(A), _ptr(B), _ptr(C), b, M, N, K)
    return C


def gemm_int64_numpy(A, B):
    """Closed form in int64: sum_k A[i,k]*B[j,k]; the result always fits int32 for K <= 65793."""
    return A.astype(np.int64) @ B.astype(np.int64).T


# --------------------------------------------------------- floating point path
def gemm_f32(A, B):
    """A (M,K), B (N,K) any float dtype -> fp32 (M,N); widened exactly, double accumulate in C."""
    A = np.ascontiguousarray(A, dtype=np.float32); B = np.ascontiguousarray(B, dtype=np.float32)
    M, K = A.shape; N = B.shape[0]
    assert B.shape[1] == K
    C = np.empty((M, N), np.float32)
    lib().orc_gemm_f32(_ptr(A), _ptr(B), _ptr(C), M, N, K)
    return C


def bmm_f32(A, B):
    A = np.ascontiguousarray(A, dtype=np.float32); B = np.ascontiguousarray(B, dtype=np.float32)
    b, M, K = A.shape; N = B.shape[1]
    C = np.empty((b, M, N), np.float32)
    lib().orc_bmm_f32(_ptr(A), _ptr(B), _ptr(C), b, M, N, K)
    return C


def conv_out_size(H, KH, stride, pad, dil):
    return (H - ((KH - 1) * dil + 1) + 2 * pad) // stride + 1


def conv2d_nhwc_f32(In, Wt, stride=1, pad=0, dil=1):
    """In (N,H,W,CI), Wt KRSC (CO,KH,KW,CI) -> (N,HO,WO,CO) fp32."""
    In = np.ascontiguousarray(In, dtype=np.float32); Wt = np.ascontiguousarray(Wt, dtype=np.float32)
    N, H, W, CI = In.shape; CO, KH, KW, CI2 = Wt.shape
    assert CI == CI2
    HO = conv_out_size(H, KH, stride, pad, dil); WO = conv_out_size(W, KW, stride, pad, dil)
    Out = np.empty((N, HO, WO, CO), np.float32)
    lib().orc_conv2d_nhwc_f32(_ptr(In), _ptr(Wt), _ptr(Out), N, H, W, CI, CO, KH, KW, stride, pad, dil)
    return Out


def conv2d_nhwc_u8s8s32(In, Wt, stride=1, pad=0, dil=1):
    """In (N,H,W,CI) uint8, Wt KRSC (CO,KH,KW,CI) int8 -> (N,HO,WO,CO) int32."""
    In = _c(In, np.uint8); Wt = _c(Wt, np.int8)
    N, H, W, CI = In.shape; CO, KH, KW, CI2 = Wt.shape
    assert CI == CI2
    HO = conv_out_size(H, KH, stride, pad, dil); WO = conv_out_size(W, KW, stride, pad, dil)
    Out = np.empty((N, HO, WO, CO), np.int32)
    lib().orc_conv2d_nhwc_u8s8s32(_ptr(In), _ptr(Wt), _ptr(Out), N, H, W, CI, CO, KH, KW, stride, pad, dil)
    return Out


def conv2d_nhwc_u8s8s32_blocked(In, Wb, stride=1, pad=0, dil=1):
    """The reference's operand shapes: Wb (CO/cb,KH,KW,CI/4,cb,4) int8 -> (N,HO,WO,CO/cb,cb) int32."""
    In = _c(In, np.uint8); Wb = _c(Wb, np.int8)
    N, H, W, CI = In.shape; OC, KH, KW, ICC, cb, four = Wb.shape
    assert four == 4 and ICC * 4 == CI
    CO = OC * cb
    HO = conv_out_size(H, KH, stride, pad, dil); WO = conv_out_size(W, KW, stride, pad, dil)
    Out = np.empty((N, HO, WO, OC, cb), np.int32)
    rc = lib().orc_conv2d_nhwc_u8s8s32_blocked(_ptr(In), _ptr(Wb), _ptr(Out), N, H, W, CI, CO, KH, KW, stride, pad, dil, cb)
    assert rc == 0
    return Out


def pack_filter_blocked(Wt, cb):
    """KRSC (CO,KH,KW,CI) -> the reference's "OhwI<cb>o4i" order (CO/cb,KH,KW,CI/4,cb,4) (conv2d_int8.py:36-50)."""
    CO, KH, KW, CI = Wt.shape
    assert CO % cb == 0 and CI % 4 == 0
    return np.ascontiguousarray(Wt.reshape(CO // cb, cb, KH, KW, CI // 4, 4).transpose(0, 2, 3, 4, 1, 5))


def unpack_filter_blocked(Wb):
    OC, KH, KW, ICC, cb, four = Wb.shape
    return np.ascontiguousarray(Wb.transpose(0, 4, 1, 2, 3, 5).reshape(OC * cb, KH, KW, ICC * 4))


def conv2d_im2col_int64_numpy(In, Wt, stride=1, pad=0, dil=1):
    """Closed form: explicit im2col matrix (numpy indexing) times the flattened filter, in int64."""
    N, H, W, CI = In.shape; CO, KH, KW, _ = Wt.shape
    HO = conv_out_size(H, KH, stride, pad, dil); WO = conv_out_size(W, KW, stride, pad, dil)
    P = np.zeros((N, H + 2 * pad, W + 2 * pad, CI), np.int64)
    P[:, pad:pad + H, pad:pad + W, :] = In
    cols = np.empty((N, HO, WO, KH, KW, CI), np.int64)
    for ry in range(KH):
        for rx in range(KW):
            cols[:, :, :, ry, rx, :] = P[:, ry * dil:ry * dil + (HO - 1) * stride + 1:stride,
                                         rx * dil:rx * dil + (WO - 1) * stride + 1:stride, :]
    return (cols.reshape(N * HO * WO, KH * KW * CI) @ Wt.astype(np.int64).reshape(CO, -1).T).reshape(N, HO, WO, CO)


def gemm_f64_numpy(A, B):
    return A.astype(np.float64) @ B.astype(np.float64).T


def bmm_f64_numpy(A, B):
    return np.einsum("bik,bjk->bij", A.astype(np.float64), B.astype(np.float64))
