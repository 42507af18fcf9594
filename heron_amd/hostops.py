"""Host-side helpers that run one template instance on torch device tensors.

torch is plumbing only (device memory and streams); every multiply goes through the C ABI.
"""
import torch

from . import backend as B


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _chk(t, dtype):
    if not (t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise ValueError("expected a contiguous CUDA tensor of %s, got %s %s" % (dtype, t.dtype, t.device))


def gemm(mod, A, Bm, out=None, group_m=8):
    """C = A @ Bm.T for A (M,K), Bm (N,K), or batched (b,M,K) x (b,N,K) -> (b,M,N)."""
    f16 = mod.desc.dtype == B.HRN_DT_F16
    _chk(A, torch.float16 if f16 else torch.uint8)
    _chk(Bm, torch.float16 if f16 else torch.int8)
    batch = A.shape[0] if A.dim() == 3 else 1
    M, K = A.shape[-2], A.shape[-1]
    N = Bm.shape[-2]
    if Bm.shape[-1] != K or (A.dim() == 3) != (Bm.dim() == 3) or (A.dim() == 3 and Bm.shape[0] != batch):
        raise ValueError("shape mismatch %s x %s" % (tuple(A.shape), tuple(Bm.shape)))
    oshape = (batch, M, N) if A.dim() == 3 else (M, N)
    if out is None:
        out = torch.empty(oshape, dtype=torch.float16 if f16 else torch.int32, device=A.device)
    p = B.gemm_problem(batch, M, N, K, group_m)
    mod.launch(p, A.data_ptr(), Bm.data_ptr(), out.data_ptr(), _stream())
    return out


def unpack_filter_blocked(Wb):
    """Blocked int8 filter (CO/b,KH,KW,CI/4,b,4) of ops/x86/conv2d_int8.py:50 -> KRSC (CO,KH,KW,CI); a one-off
    reorder of the weights on the device."""
    OC, KH, KW, ICC, cb, four = Wb.shape
    if four != 4:
        raise ValueError("expected (CO/b,KH,KW,CI/4,b,4), got %s" % (tuple(Wb.shape),))
    return Wb.permute(0, 4, 1, 2, 3, 5).reshape(OC * cb, KH, KW, ICC * 4).contiguous()


def conv2d_nhwc(mod, X, Wt, stride=1, pad=0, dil=1, out=None, group_m=8):
    """X (N,H,W,CI), Wt KRSC (CO,KH,KW,CI) -> (N,HO,WO,CO): fp16 -> fp16, or uint8 x int8 -> int32."""
    f16 = mod.desc.dtype == B.HRN_DT_F16
    _chk(X, torch.float16 if f16 else torch.uint8)
    _chk(Wt, torch.float16 if f16 else torch.int8)
    N, H, W, CI = X.shape
    CO, KH, KW, CI2 = Wt.shape
    if CI != CI2:
        raise ValueError("channel mismatch")
    p = B.conv2d_problem(N, H, W, CI, CO, KH, KW, stride, pad, dil, group_m)
    ho = (H - ((KH - 1) * dil + 1) + 2 * pad) // stride + 1
    wo = (W - ((KW - 1) * dil + 1) + 2 * pad) // stride + 1
    if out is None:
        out = torch.empty((N, ho, wo, CO), dtype=torch.float16 if f16 else torch.int32, device=X.device)
    mod.launch(p, X.data_ptr(), Wt.data_ptr(), out.data_ptr(), _stream())
    return out
