"""Host-side helpers that run one template instance on torch device tensors.

torch is plumbing only (device memory and streams); every multiply goes through the C ABI.
"""
import torch

from . import backend as B


def _stream():
    return torch.cuda.current_stream().cuda_stream


# While an OperatorPlan is being recorded, every library call of this module is also appended here (callable, arguments):
# replaying the list repeats the device work of the call without its Python and torch bookkeeping.
_recording = None


_keepalive = None


def _new(maker, *args, **kwargs):
    """A fresh tensor; while a plan is recorded it is kept alive with the plan (the recorded calls hold addresses)."""
    t = maker(*args, **kwargs)
    if _keepalive is not None:
        _keepalive.append(t)
    return t


def _do(fn, *args):
    if _recording is not None:
        _recording.append((fn, args))
    return fn(*args)


def _chk(t, dtype):
    if not (t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise ValueError("expected a contiguous CUDA tensor of %s, got %s %s" % (dtype, t.dtype, t.device))


def column_sums(Bm):
    """Column sums of an int8 operand (N,K) / (b,N,K) / KRSC filter (CO,KH,KW,CI): int32 (N,) / (b,N) / (CO,).  What a
    ``colsum`` instance takes with the weights; with fixed weights it is computed once."""
    _chk(Bm, torch.int8)
    if Bm.dim() == 4:
        n, k, batch = Bm.shape[0], Bm.shape[1] * Bm.shape[2] * Bm.shape[3], 1
    else:
        n, k, batch = Bm.shape[-2], Bm.shape[-1], (Bm.shape[0] if Bm.dim() == 3 else 1)
    out = _new(torch.empty, (batch, n) if Bm.dim() == 3 else (n,), dtype=torch.int32, device=Bm.device)
    B.colsum_s8(Bm.data_ptr(), out.data_ptr(), batch, n, k, stream=_stream())
    return out


def gemm(mod, A, Bm, out=None, group_m=8, split_k=0, bsum=None):
    """C = A @ Bm.T for A (M,K), Bm (N,K), or batched (b,M,K) x (b,N,K) -> (b,M,N).  ``split_k`` is the number of
    K slices for a split-K instance (the module supplies the workspace).  ``bsum``: the column sums of Bm
    (``column_sums``) for a ``colsum`` instance; computed on the spot when absent."""
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
        out = _new(torch.empty, oshape, dtype=torch.float16 if f16 else torch.int32, device=A.device)
    p = B.gemm_problem(batch, M, N, K, group_m, split_k)
    if bsum is not None and mod.desc.colsum:
        _chk(bsum, torch.int32)
        if bsum.numel() != batch * N:
            raise ValueError("bsum holds %d sums, B has %d columns" % (bsum.numel(), batch * N))
        p.bsum = bsum.data_ptr()
    _do(mod.launch, p, A.data_ptr(), Bm.data_ptr(), out.data_ptr(), _stream())
    return out


def unpack_filter_blocked(Wb):
    """Blocked int8 filter (CO/b,KH,KW,CI/4,b,4) of ops/x86/conv2d_int8.py:50 -> KRSC (CO,KH,KW,CI); a one-off
    reorder of the weights on the device."""
    OC, KH, KW, ICC, cb, four = Wb.shape
    if four != 4:
        raise ValueError("expected (CO/b,KH,KW,CI/4,b,4), got %s" % (tuple(Wb.shape),))
    return Wb.permute(0, 4, 1, 2, 3, 5).reshape(OC * cb, KH, KW, ICC * 4).contiguous()


def conv2d_nhwc(mod, X, Wt, stride=1, pad=0, dil=1, out=None, group_m=8, split_k=0, bsum=None):
    """X (N,H,W,CI), Wt KRSC (CO,KH,KW,CI) -> (N,HO,WO,CO): fp16 -> fp16, or uint8 x int8 -> int32."""
    f16 = mod.desc.dtype == B.HRN_DT_F16
    _chk(X, torch.float16 if f16 else torch.uint8)
    _chk(Wt, torch.float16 if f16 else torch.int8)
    N, H, W, CI = X.shape
    CO, KH, KW, CI2 = Wt.shape
    if CI != CI2:
        raise ValueError("channel mismatch")
    p = B.conv2d_problem(N, H, W, CI, CO, KH, KW, stride, pad, dil, group_m, split_k)
    (sh, sw), (ph, pw), (dh, dw) = B._pair(stride), B._pair(pad), B._pair(dil)
    ho = (H - ((KH - 1) * dh + 1) + 2 * ph) // sh + 1
    wo = (W - ((KW - 1) * dw + 1) + 2 * pw) // sw + 1
    if out is None:
        out = _new(torch.empty, (N, ho, wo, CO), dtype=torch.float16 if f16 else torch.int32, device=X.device)
    if bsum is not None and mod.desc.colsum:
        _chk(bsum, torch.int32)
        if bsum.numel() != CO:
            raise ValueError("bsum holds %d sums, the filter has %d output channels" % (bsum.numel(), CO))
        p.bsum = bsum.data_ptr()
    _do(mod.launch, p, X.data_ptr(), Wt.data_ptr(), out.data_ptr(), _stream())
    return out


# ----------------------------------------------------------------------------------------------
# Operand adapters: the reference declares several operators as "injective pre-stage + matrix product"
# (layout changes, padding, constant right-hand sides).  An adapter is that pre-stage: it maps the caller's
# tensors, in the reference's layouts, to the template's operands (A (M,K) / B (N,K), or NHWC / KRSC) and
# maps the result back.  They only move, pad or generate data; every multiply-accumulate is the kernel's.
def _pad_last(t, to):
    """``t`` with its last axis zero-padded to ``to`` elements, contiguous."""
    c = t.shape[-1]
    if c == to:
        return t.contiguous()
    if t.is_cuda and t.is_contiguous() and t.element_size() in (1, 2) and (to * t.element_size()) % 16 == 0:
        out = _new(torch.empty, t.shape[:-1] + (to,), dtype=t.dtype, device=t.device)
        _do(B.pad_rows, t.data_ptr(), out.data_ptr(), t.numel() // c, c, to, t.element_size(), _stream())
        return out
    return torch.nn.functional.pad(t, (0, to - c)).contiguous()


def _native_ok(t):
    return t.is_cuda and t.is_contiguous() and t.element_size() in (1, 2, 4)


def _gather(src, out, dst_dim, coords, dst_stride=None, dst_live=None, op=B.GATHER_COPY, aux=None):
    """One pass of the library's affine gather from ``src`` into ``out`` (both contiguous device tensors; see
    backend.make_gather for ``coords``)."""
    g = B.make_gather(src.element_size(), dst_dim, coords, dst_stride, dst_live, op)
    _do(B.gather_nd, g, src.data_ptr(), out.data_ptr(), aux.data_ptr() if aux is not None else None, _stream())
    return out


def _channels_last(x3, cp=None):
    """(N, C, L) -> (N, L, cp): channels become the last axis, zero-padded to ``cp`` (one pass of the library)."""
    N, C, L = x3.shape
    cp = cp or C
    if _native_ok(x3) and N <= 65535 and L > 0:
        out = _new(torch.empty, (N, L, cp), dtype=x3.dtype, device=x3.device)
        _do(B.transpose_pad, x3.data_ptr(), out.data_ptr(), N, C, L, cp, x3.element_size(), _stream())
        return out
    return _pad_last(x3.permute(0, 2, 1), cp)


def _channels_first(y3):
    """(N, L, C) -> (N, C, L)."""
    N, L, C = y3.shape
    if _native_ok(y3) and N <= 65535 and L > 0:
        out = _new(torch.empty, (N, C, L), dtype=y3.dtype, device=y3.device)
        _do(B.transpose_pad, y3.data_ptr(), out.data_ptr(), N, L, C, L, y3.element_size(), _stream())
        return out
    return y3.permute(0, 2, 1).contiguous()


# Every adapter has two halves: ``act`` maps the activation input(s) to the kernel's A operand and is needed on every
# call; ``const`` maps the constant input (filter, vector) - or nothing but the shapes - to the kernel's B operand and is
# needed once per set of weights (run_operator caches it when asked to).
def _act_identity(info, A, Bm):
    return A


def _const_identity(info, A, Bm):
    return Bm


def _act_pad_k(info, A, *_):
    return _pad_last(A, info['gemm_view']['K'])


def _const_gemv(info, A, b):
    g = info['gemm_view']
    Bp = _new(torch.zeros, (g['N'], g['K']), dtype=b.dtype, device=b.device)
    Bp[0, :b.shape[-1]] = b.reshape(-1)
    return Bp


def _const_scan(info, A):
    g = info['gemm_view']
    n = torch.arange(g['N'], device=A.device).unsqueeze(1)
    k = torch.arange(g['K'], device=A.device).unsqueeze(0)
    T = (n > k).to(torch.float16 if info['kind'] == 'f16' else torch.int8)
    T[:, A.shape[-1]:] = 0
    return T


def _channel_major(info, In, mean=None):
    """(N,C,H,W) -> (C, K) with K = N*H*W zero-padded to the kernel's K; with ``mean`` (same shape as ``In``) every
    element becomes (x - mean)^2 on the way (fp16, both steps rounded as separate fp16 tensor operations would)."""
    N, C, H, W = In.shape
    K = info['gemm_view']['K']
    if not (_native_ok(In) and (mean is None or (_native_ok(mean) and In.dtype == torch.float16))):
        if mean is not None:
            d = In - mean
            In = d * d
        return _pad_last(In.permute(1, 0, 2, 3).reshape(C, N * H * W), K)
    out = _new(torch.empty if K == N * H * W else torch.zeros, (C, K), dtype=In.dtype, device=In.device)
    return _gather(In, out, (C, N, H * W), [(N, C * H * W, {1: 1}), (C, H * W, {0: 1}), (H * W, 1, {2: 1})],
                   dst_stride=(K, H * W, 1), op=B.GATHER_CENTER_SQUARE if mean is not None else B.GATHER_COPY, aux=mean)


def _act_mean(info, In, *_):
    return _channel_major(info, In)


def _const_mean(info, In, *_):
    g = info['gemm_view']
    N, C, H, W = In.shape
    Bm = _new(torch.zeros, (g['N'], g['K']), dtype=In.dtype, device=In.device)
    Bm[0, :N * H * W] = 1.0 / (N * H * W)
    return Bm


def _act_var(info, In, Mean):
    if tuple(Mean.shape) != tuple(In.shape) or Mean.dtype != In.dtype:
        raise ValueError("var takes a Mean of In's shape and type, got %s for %s" % (tuple(Mean.shape), tuple(In.shape)))
    return _channel_major(info, In, Mean)


def _cpad(info):
    return info['conv']['CI']


def _act_c1d_nwc(info, X, F):             # (N,W,CI)
    return _pad_last(X, _cpad(info)).unsqueeze(1)


def _const_c1d_nwc(info, X, F):           # (K,CI,CO)
    return _pad_last(F.permute(2, 0, 1), _cpad(info)).unsqueeze(1).contiguous()


def _act_c1d_ncw(info, X, F):             # (N,CI,W)
    return _channels_last(X, _cpad(info)).unsqueeze(1)


def _const_c1d_ncw(info, X, F):           # (CO,CI,KW)
    return _pad_last(F.permute(0, 2, 1), _cpad(info)).unsqueeze(1).contiguous()


def _act_nchw(info, X, F):                # (N,CI,H,W)
    N, CI, H, W = X.shape
    return _channels_last(X.reshape(N, CI, H * W), _cpad(info)).reshape(N, H, W, _cpad(info))


def _const_oihw(info, X, F):              # (CO,CI,KH,KW)
    return _pad_last(F.permute(0, 2, 3, 1), _cpad(info))


def _act_nhwc(info, X, F):                # (N,H,W,CI), CI possibly short of a whole 16-byte chunk
    return _pad_last(X, _cpad(info))


def _const_krsc(info, X, F):              # (CO,KH,KW,CI)
    return _pad_last(F, _cpad(info))


def _const_hwio(info, X, F):              # (KH,KW,CI,CO)
    return _pad_last(F.permute(3, 0, 1, 2), _cpad(info))


def _act_c3d_ndhwc(info, X, F):           # (N,D,H,W,CI)
    dp = info['depth']
    N, D, H, W, CI = X.shape
    KD, DO, sd, pd, dd = dp['KD'], dp['DO'], dp['stride'], dp['pad'], dp['dil']
    cip = info['conv']['CI'] // KD
    if _native_ok(X):
        # depth taps side by side on the channel axis: channel block kd of output slice z is input slice z*sd + kd*dd - pd
        out = _new(torch.empty, (N * DO, H, W, KD * cip), dtype=X.dtype, device=X.device)
        return _gather(X, out, (N, DO, H * W, KD, cip),
                       [(N, D * H * W * CI, {0: 1}), (D, H * W * CI, {1: sd, 3: dd}, -pd), (H * W, CI, {2: 1}), (CI, 1, {4: 1})],
                       dst_live=(N, DO, H * W, KD, CI))
    Xp = _new(torch.zeros, (N, D + 2 * pd, H, W, cip), dtype=X.dtype, device=X.device)
    Xp[:, pd:pd + D, :, :, :CI] = X
    # depth taps side by side on the channel axis: channel block kd of output slice z is input slice z*sd + kd*dd
    cols = torch.stack([Xp[:, kd * dd: kd * dd + (DO - 1) * sd + 1: sd] for kd in range(KD)], dim=4)
    return cols.reshape(N * DO, H, W, KD * cip).contiguous()


def _const_c3d_dhwio(info, X, F):         # (KD,KH,KW,CI,CO)
    KD = info['depth']['KD']
    cip = info['conv']['CI'] // KD
    Fp = _pad_last(F.permute(4, 1, 2, 0, 3), cip)                    # (CO,KH,KW,KD,cip)
    return Fp.reshape(Fp.shape[0], Fp.shape[1], Fp.shape[2], KD * cip).contiguous()


def _act_c3d_ncdhw(info, X, F):           # (N,CI,D,H,W)
    N, CI, D, H, W = X.shape
    return _act_c3d_ndhwc(info, _channels_last(X.reshape(N, CI, D * H * W)).reshape(N, D, H, W, CI), F)


def _const_c3d_oidhw(info, X, F):         # (CO,CI,KD,KH,KW)
    return _const_c3d_dhwio(info, X, F.permute(2, 3, 4, 1, 0))


def _act_t2d_nchw(info, X, F):            # (N,CI,H,W): zero-expanded by the stride and padded, channels last
    t = info['transposed']
    c = info['conv']
    N, CI, H, W = X.shape
    s = t['stride']
    top = (c['KH'] - 1) * t['dil'] - t['pad']
    left = (c['KW'] - 1) * t['dil'] - t['pad']
    if _native_ok(X) and N <= 65535:
        # channels last (and padded) first, then one pass that writes every pixel of the expanded image: input pixel
        # ((y - top) / s, (x - left) / s) where both divide, zero elsewhere
        Xc = _channels_last(X.reshape(N, CI, H * W), c['CI'])
        Xe = _new(torch.empty, (N, c['H'], c['W'], c['CI']), dtype=X.dtype, device=X.device)
        return _gather(Xc, Xe, (N, c['H'], c['W'], c['CI']),
                       [(N, H * W * c['CI'], {0: 1}), (H, W * c['CI'], {1: 1}, -top, s), (W, c['CI'], {2: 1}, -left, s),
                        (c['CI'], 1, {3: 1})])
    Xe = _new(torch.zeros, (N, c['H'], c['W'], c['CI']), dtype=X.dtype, device=X.device)
    if s > 1:
        # channels last (and padded) first, so that the strided scatter moves whole pixels (stride 2: 137 -> 70 us end
        # to end on 16x56x56x64); with stride 1 the permuted assignment is one pass and an extra launch only costs
        Xe[:, top: top + (H - 1) * s + 1: s, left: left + (W - 1) * s + 1: s, :] = \
            _channels_last(X.reshape(N, CI, H * W), c['CI']).reshape(N, H, W, c['CI'])
    else:
        Xe[:, top: top + H, left: left + W, :CI] = X.permute(0, 2, 3, 1)
    return Xe


def _act_dep(info, X, F):                 # (N,C,H,W): the 3x3 windows as 4x4 = 16 taps per pixel and channel
    d = info['dep']
    N, C, H, W = X.shape
    s, p, HO, WO = d['stride'], d['pad'], d['HO'], d['WO']
    if _native_ok(X):
        A = _new(torch.empty, (C, N * HO * WO, 16), dtype=X.dtype, device=X.device)
        return _gather(X, A, (C, N, HO, WO, 4, 4),
                       [(N, C * H * W, {1: 1}), (C, H * W, {0: 1}), (H, W, {2: s, 4: 1}, -p), (W, 1, {3: s, 5: 1}, -p)],
                       dst_live=(C, N, HO, WO, 3, 3))
    Xp = _new(torch.zeros, (N, C, H + 2 * p + 1, W + 2 * p + 1), dtype=X.dtype, device=X.device)
    Xp[:, :, p:p + H, p:p + W] = X
    A = _new(torch.zeros, (C, N, HO, WO, 4, 4), dtype=X.dtype, device=X.device)
    for r in range(3):
        for q in range(3):
            A[:, :, :, :, r, q] = Xp[:, :, r: r + (HO - 1) * s + 1: s, q: q + (WO - 1) * s + 1: s].permute(1, 0, 2, 3)
    return A.reshape(C, N * HO * WO, 16)


def _const_dep(info, X, F):               # (K,3,3)
    d = info['dep']
    C, mult, NP = X.shape[1], d['mult'], d['NP']
    Bm = _new(torch.zeros, (C, NP, 4, 4), dtype=F.dtype, device=F.device)
    Bm[:, :mult, :3, :3] = F.reshape(C, mult, 3, 3)
    return Bm.reshape(C, NP, 16)


def _fin_dep(info, Cm):                   # (C, N*HO*WO, NP) -> (N, C, NP, HO, WO)
    d = info['dep']
    C, N, HW, NP = d['C'], d['N'], d['HO'] * d['WO'], d['NP']
    if _native_ok(Cm):
        out = _new(torch.empty, (N, C, NP, d['HO'], d['WO']), dtype=Cm.dtype, device=Cm.device)
        return _gather(Cm, out, (N, C, NP, HW), [(C, N * HW * NP, {1: 1}), (N, HW * NP, {0: 1}), (HW, NP, {3: 1}), (NP, 1, {2: 1})])
    return Cm.reshape(d['C'], d['N'], d['HO'], d['WO'], d['NP']).permute(1, 0, 4, 2, 3).contiguous()


def _fin_identity(info, C):
    return C


def _fin_c1d_nwc(info, C):                # (N,1,WO,CO) -> (N,WO,CO)
    return C.squeeze(1)


def _fin_c1d_ncw(info, C):                # -> (N,CO,WO)
    return _channels_first(C.squeeze(1))


def _fin_nchw(info, C):                   # (N,HO,WO,CO) -> (N,CO,HO,WO)
    N, HO, WO, CO = C.shape
    return _channels_first(C.reshape(N, HO * WO, CO)).reshape(N, CO, HO, WO)


def _fin_c3d_ndhwc(info, C):              # (N*DO,HO,WO,CO) -> (N,DO,HO,WO,CO)
    dp = info['depth']
    return C.reshape(dp['N'], dp['DO'], C.shape[1], C.shape[2], C.shape[3])


def _fin_c3d_ncdhw(info, C):              # -> (N,CO,DO,HO,WO)
    Y = _fin_c3d_ndhwc(info, C)
    N, DO, HO, WO, CO = Y.shape
    return _channels_first(Y.reshape(N, DO * HO * WO, CO)).reshape(N, CO, DO, HO, WO)


ADAPTERS = {
    # name: (activation half, constant half, result reorder)
    'identity': (_act_identity, _const_identity, _fin_identity),
    'gemv': (_act_pad_k, _const_gemv, _fin_identity),
    'scan': (_act_pad_k, _const_scan, _fin_identity),
    'mean': (_act_mean, _const_mean, _fin_identity),
    'var': (_act_var, _const_mean, _fin_identity),
    'c1d_nwc': (_act_c1d_nwc, _const_c1d_nwc, _fin_c1d_nwc),
    'c1d_ncw': (_act_c1d_ncw, _const_c1d_ncw, _fin_c1d_ncw),
    'c2d_nchw': (_act_nchw, _const_oihw, _fin_nchw),
    'c2d_hwio': (_act_nhwc, _const_hwio, _fin_identity),
    'c2d_krsc': (_act_nhwc, _const_krsc, _fin_identity),
    'c3d_ndhwc': (_act_c3d_ndhwc, _const_c3d_dhwio, _fin_c3d_ndhwc),
    'c3d_ncdhw': (_act_c3d_ncdhw, _const_c3d_oidhw, _fin_c3d_ncdhw),
    't2d_nchw': (_act_t2d_nchw, _const_oihw, _fin_nchw),
    'dep': (_act_dep, _const_dep, _fin_dep),
}


# adapters whose ACTIVATION operand passes through unchanged when its channel count is a whole 16-byte chunk: the
# caller's tensor is already channels-last, only the (constant) filter is reordered once
ACTIVATION_AS_IS = ('identity', 'c1d_nwc', 'c2d_hwio', 'c2d_krsc')


def prepare_constant(info, inputs):
    """The kernel's B operand of an operator: the reordered / padded filter or the generated right-hand side.  It
    depends on the weights and the shapes only, so a caller with fixed weights prepares it once."""
    return ADAPTERS[info.get('adapter', 'identity')][1](info, *inputs)


def run_operator(mod, info, inputs, group_m=8, split_k=0, constant=None, bsum=None):
    """Runs one operator of the registry on device tensors given in the reference's own layouts.

    ``info`` is the dictionary the operator definition handed to ``ctx.set_info``; ``mod`` an instance of the
    template that matches its kind and operator; ``constant`` a B operand from ``prepare_constant`` (made here when
    absent); ``bsum`` its column sums (``column_sums``) for a ``colsum`` instance."""
    act, const, fin = ADAPTERS[info.get('adapter', 'identity')]
    A = act(info, *inputs)
    Bm = const(info, *inputs) if constant is None else constant
    if info['operator'] == 'conv2d_nhwc':
        c = info['conv']
        C = conv2d_nhwc(mod, A, Bm, (c['stride'], c['stride_w']), (c['pad'], c['pad_w']), (c['dil'], c['dil_w']),
                        group_m=group_m, split_k=split_k, bsum=bsum)
    else:
        C = gemm(mod, A, Bm, group_m=group_m, split_k=split_k, bsum=bsum)
    return fin(info, C)


class OperatorPlan:
    """One operator on fixed device tensors, recorded once and replayed: ``run()`` repeats the library passes and the
    kernel launch of ``run_operator`` (same order, same stream, same buffers) without allocating, without building
    index maps and without any torch call, and returns the same result tensor every time.  What a caller with
    preallocated buffers pays per call.  The inputs are bound by address: new data goes into the same tensors.

    A recording is only valid if every byte the operator moves is moved by a recorded call.  ``validate`` checks that:
    the activation is changed in place, the operator is run eagerly and by replay, and both results must agree."""

    def __init__(self, mod, info, inputs, group_m=8, split_k=0, constant=None, validate=True):
        global _recording, _keepalive
        if _recording is not None:
            raise RuntimeError("an operator plan is already being recorded")
        self.inputs = list(inputs)
        self.constant = prepare_constant(info, inputs) if constant is None else constant
        self.bsum = column_sums(self.constant) if mod.desc.colsum else None
        self._keep = (mod, info)
        stream = _stream()
        _recording, _keepalive = steps, buffers = [], []
        try:
            self.out = run_operator(mod, info, self.inputs, group_m, split_k, self.constant, self.bsum)
        finally:
            _recording = _keepalive = None
        self.steps, self.buffers = steps, buffers
        self.stream = stream
        if any(a[-1] != stream for _, a in steps):
            raise RuntimeError("the recorded passes ran on more than one stream")
        if validate:
            x = self.inputs[0]
            saved = x.clone()
            if x.dtype == torch.float16:
                x.mul_(-0.5)
            else:
                x.copy_(255 - x if x.dtype == torch.uint8 else -(x.clamp(min=-127)))
            want = run_operator(mod, info, self.inputs, group_m, split_k, self.constant, self.bsum).clone()
            self.out.zero_()
            got = self.run()
            ok = torch.equal(got, want)
            x.copy_(saved)
            self.run()
            if not ok:
                raise RuntimeError("operator plan: the replay does not reproduce the operator (a pre-stage of adapter "
                                   "%r moves data outside the recorded passes)" % info.get('adapter', 'identity'))

    def run(self):
        if _stream() != self.stream:
            raise RuntimeError("an operator plan replays on the stream it was recorded on")
        for fn, args in self.steps:
            fn(*args)
        return self.out

