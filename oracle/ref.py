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
        L.orc_conv2d_nhwc_f32.argtypes = [_p, _p, _p] + [_i64] * 13
        L.orc_conv2d_nhwc_u8s8s32.argtypes = [_p, _p, _p] + [_i64] * 13
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


def _pair(v):
    return (int(v), int(v)) if isinstance(v, (int, np.integer)) else (int(v[0]), int(v[1]))


def conv_out_size(H, KH, stride, pad, dil):
    return (H - ((KH - 1) * dil + 1) + 2 * pad) // stride + 1


def conv2d_nhwc_f32(In, Wt, stride=1, pad=0, dil=1):
    """In (N,H,W,CI), Wt KRSC (CO,KH,KW,CI) -> (N,HO,WO,CO) fp32."""
    In = np.ascontiguousarray(In, dtype=np.float32); Wt = np.ascontiguousarray(Wt, dtype=np.float32)
    N, H, W, CI = In.shape; CO, KH, KW, CI2 = Wt.shape
    assert CI == CI2
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(pad), _pair(dil)
    HO = conv_out_size(H, KH, sh, ph, dh); WO = conv_out_size(W, KW, sw, pw, dw)
    Out = np.empty((N, HO, WO, CO), np.float32)
    lib().orc_conv2d_nhwc_f32(_ptr(In), _ptr(Wt), _ptr(Out), N, H, W, CI, CO, KH, KW, sh, sw, ph, pw, dh, dw)
    return Out


def conv2d_nhwc_u8s8s32(In, Wt, stride=1, pad=0, dil=1):
    """In (N,H,W,CI) uint8, Wt KRSC (CO,KH,KW,CI) int8 -> (N,HO,WO,CO) int32."""
    In = _c(In, np.uint8); Wt = _c(Wt, np.int8)
    N, H, W, CI = In.shape; CO, KH, KW, CI2 = Wt.shape
    assert CI == CI2
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(pad), _pair(dil)
    HO = conv_out_size(H, KH, sh, ph, dh); WO = conv_out_size(W, KW, sw, pw, dw)
    Out = np.empty((N, HO, WO, CO), np.int32)
    lib().orc_conv2d_nhwc_u8s8s32(_ptr(In), _ptr(Wt), _ptr(Out), N, H, W, CI, CO, KH, KW, sh, sw, ph, pw, dh, dw)
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


# ------------------------------------------------- operators declared as a pre-stage + product
# Each follows the te.compute declaration of the reference operator it names, in float64 (or int64),
# in the reference's own operand layouts.  tests/test_oracle.py pins them against numpy / torch library
# routines (cumsum, mean, conv1d, conv2d, conv3d, conv_transpose2d).
def _wide(a):
    return a.astype(np.int64) if a.dtype.kind in "iu" else a.astype(np.float64)


def gemv_ref(A, b):
    """ops/cuda/gemv.py:4-31: out (M,8) = A (M,K) x pad8(b (1,K)); only column 0 is non-zero."""
    out = np.zeros((A.shape[0], 8), _wide(A).dtype)
    for i in range(A.shape[0]):
        out[i, 0] = (_wide(A[i]) * _wide(b.reshape(-1))).sum()
    return out


def scan_ref(A, N):
    """ops/cuda/scan.py:4-23: out[m,n] = sum_k A[m,k] * T[n,k] with T[n,k] = 0 if n <= k else 1."""
    M, K = A.shape
    T = np.zeros((N, K), _wide(A).dtype)
    for n in range(N):
        for k in range(K):
            T[n, k] = 0 if n <= k else 1
    return _wide(A) @ T.T


def mean_ref(In):
    """ops/cuda/mean.py:4-31: A[c, j] = In[j // (H*W), c, j % (H*W) // W, j % W]; B[0, :] = 1/(N*H*W); out (C,8).
    The constant is rounded to the input precision as the declaration's tvm.tir.const(..., in_dtype) does."""
    N, C, H, W = In.shape
    K = N * H * W
    A = np.empty((C, K), np.float64)
    for j in range(K):
        A[:, j] = In[j // (H * W), :, j % (H * W) // W, j % W]
    out = np.zeros((C, 8), np.float64)
    out[:, 0] = A.sum(1) * float(In.dtype.type(1.0 / K))
    return out


def var_ref(In, Mean):
    """ops/cuda/var.py:4-40: mean_ref of (In - Mean)**2, the difference and square taken in the input precision."""
    d = (In - Mean).astype(In.dtype)
    return mean_ref((d * d).astype(In.dtype))


def conv1d_nwc_ref(X, F, stride, pad, dil):
    """ops/cuda/conv1d.py:109-151: X (N,W,CI), F (K,CI,CO) -> (N,WO,CO)."""
    N, W, CI = X.shape
    K, _, CO = F.shape
    WO = conv_out_size(W, K, stride, pad, dil)
    P = np.zeros((N, W + 2 * pad, CI), _wide(X).dtype)
    P[:, pad:pad + W] = X
    out = np.zeros((N, WO, CO), P.dtype)
    for rw in range(K):
        out += P[:, rw * dil: rw * dil + (WO - 1) * stride + 1: stride] @ _wide(F[rw])
    return out


def conv1d_ncw_ref(X, F, stride, pad, dil):
    """ops/cuda/conv1d.py:11-72: X (N,CI,W), F (CO,CI,KW) -> (N,CO,WO)."""
    return conv1d_nwc_ref(X.transpose(0, 2, 1), F.transpose(2, 1, 0), stride, pad, dil).transpose(0, 2, 1)


def conv2d_nchw_ref(X, F, stride, pad, dil=1):
    """ops/cuda/conv2d.py:9-100: X (N,CI,H,W), F (CO,CI,KH,KW) -> (N,CO,HO,WO)."""
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(pad), _pair(dil)
    N, CI, H, W = X.shape
    CO, _, KH, KW = F.shape
    HO, WO = conv_out_size(H, KH, sh, ph, dh), conv_out_size(W, KW, sw, pw, dw)
    P = np.zeros((N, CI, H + 2 * ph, W + 2 * pw), _wide(X).dtype)
    P[:, :, ph:ph + H, pw:pw + W] = X
    out = np.zeros((N, CO, HO, WO), P.dtype)
    for ry in range(KH):
        for rx in range(KW):
            patch = P[:, :, ry * dh: ry * dh + (HO - 1) * sh + 1: sh, rx * dw: rx * dw + (WO - 1) * sw + 1: sw]
            out += np.einsum("nchw,oc->nohw", patch, _wide(F[:, :, ry, rx]))
    return out


def dil_nhwc_ref(X, F, stride, pad, dil):
    """ops/cuda/dil.py:8-68: X (N,H,W,CI), F (KH,KW,CI,CO) -> (N,HO,WO,CO)."""
    return conv2d_nchw_ref(X.transpose(0, 3, 1, 2), F.transpose(3, 2, 0, 1), stride, pad, dil).transpose(0, 2, 3, 1)


def conv3d_ndhwc_ref(X, F, stride, pad, dil):
    """ops/cuda/conv3d.py:117-197: X (N,D,H,W,CI), F (KD,KH,KW,CI,CO) -> (N,DO,HO,WO,CO)."""
    t3 = lambda v: (int(v),) * 3 if isinstance(v, (int, np.integer)) else tuple(int(x) for x in v)
    (sd, sh, sw), (pd, ph, pw), (dd, dh, dw) = t3(stride), t3(pad), t3(dil)
    N, D, H, W, CI = X.shape
    KD, KH, KW, _, CO = F.shape
    DO, HO, WO = conv_out_size(D, KD, sd, pd, dd), conv_out_size(H, KH, sh, ph, dh), conv_out_size(W, KW, sw, pw, dw)
    P = np.zeros((N, D + 2 * pd, H + 2 * ph, W + 2 * pw, CI), _wide(X).dtype)
    P[:, pd:pd + D, ph:ph + H, pw:pw + W] = X
    out = np.zeros((N, DO, HO, WO, CO), P.dtype)
    for rz in range(KD):
        for ry in range(KH):
            for rx in range(KW):
                patch = P[:, rz * dd: rz * dd + (DO - 1) * sd + 1: sd, ry * dh: ry * dh + (HO - 1) * sh + 1: sh,
                          rx * dw: rx * dw + (WO - 1) * sw + 1: sw]
                out += patch @ _wide(F[rz, ry, rx])
    return out


def conv3d_ncdhw_ref(X, F, stride, pad, dil=1):
    """ops/cuda/conv3d.py:10-82: X (N,CI,D,H,W), F (CO,CI,KD,KH,KW) -> (N,CO,DO,HO,WO)."""
    return conv3d_ndhwc_ref(X.transpose(0, 2, 3, 4, 1), F.transpose(2, 3, 4, 1, 0), stride, pad, dil).transpose(0, 4, 1, 2, 3)


def conv2d_transposed_nchw_ref(X, F, stride, pad, dil, outpad):
    """ops/cuda/conv2d_transposed.py:59-133: X (N,CI,H,W), F (CO,CI,KH,KW).  zero_expand2d by the stride,
    zero_pad2d by dilated_K-1-pad (+outpad after), then out[n,c,p,q] = sum Padded[n,ci,p+r*dil,q+s*dil] F[c,ci,r,s]
    with H_O = (H-1)*stride - 2*pad + dilated_KH + outpad."""
    N, CI, H, W = X.shape
    CO, _, KH, KW = F.shape
    dkh, dkw = (KH - 1) * dil + 1, (KW - 1) * dil + 1
    HO = (H - 1) * stride - 2 * pad + dkh + outpad
    WO = (W - 1) * stride - 2 * pad + dkw + outpad
    E = np.zeros((N, CI, (H - 1) * stride + 1, (W - 1) * stride + 1), _wide(X).dtype)
    E[:, :, ::stride, ::stride] = X
    t, l = dkh - 1 - pad, dkw - 1 - pad
    P = np.zeros((N, CI, E.shape[2] + 2 * t + outpad, E.shape[3] + 2 * l + outpad), E.dtype)
    P[:, :, t:t + E.shape[2], l:l + E.shape[3]] = E
    out = np.zeros((N, CO, HO, WO), E.dtype)
    for r in range(KH):
        for s in range(KW):
            out += np.einsum("nchw,oc->nohw", P[:, :, r * dil: r * dil + HO, s * dil: s * dil + WO], _wide(F[:, :, r, s]))
    return out


def depthwise_conv2d_ref(X, F, stride, pad):
    """ops/cuda/dep.py:9-91: X (N,C,H,W), F (K,3,3) with K = mult*C -> (N, C, ceil8(mult), HO, WO);
    out[n,c,m,p,q] = sum_{r,s<3} Pad(X)[n,c,p*stride+r,q*stride+s] * F[c*mult+m,r,s], rows m >= mult are zero."""
    N, C, H, W = X.shape
    K = F.shape[0]
    mult = K // C
    NP = (mult + 7) // 8 * 8
    HO, WO = (H - 3 + 2 * pad) // stride + 1, (W - 3 + 2 * pad) // stride + 1
    P = np.zeros((N, C, H + 2 * pad, W + 2 * pad), _wide(X).dtype)
    P[:, :, pad:pad + H, pad:pad + W] = X
    out = np.zeros((N, C, NP, HO, WO), P.dtype)
    Fw = _wide(F).reshape(C, mult, 3, 3)
    for r in range(3):
        for s in range(3):
            patch = P[:, :, r: r + (HO - 1) * stride + 1: stride, s: s + (WO - 1) * stride + 1: stride]
            out[:, :, :mult] += patch[:, :, None] * Fw[None, :, :, r, s, None, None]
    return out
