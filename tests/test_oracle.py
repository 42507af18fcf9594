"""Pins the CPU oracle (test infrastructure) independently of the HIP path.

The reference holds no golden output for its operators, so each oracle function is pinned by
checks that a plausible mistake (dropped term, wrong sign/index, transposed operand) fails:
brute-force Python loops on tiny inputs, numpy int64 closed form, hardware ``vpdpbusd`` path vs the
scalar loop, extreme-value closed forms, torch's CPU conv2d, identities and linearity.
"""
import numpy as np
import pytest
import torch

import oracle
from heron_amd import workloads


def brute_gemm(A, B):
    M, K = A.shape
    N = B.shape[0]
    C = [[0] * N for _ in range(M)]
    for i in range(M):
        for j in range(N):
            s = 0
            for k in range(K):
                s += int(A[i, k]) * int(B[j, k])
            C[i][j] = s
    return np.array(C)


def test_int_gemm_against_brute_force_and_numpy():
    rng = np.random.default_rng(0)
    A = rng.integers(0, 256, (5, 12), dtype=np.uint8)
    B = rng.integers(-128, 128, (7, 12), dtype=np.int8)       # non-square: a transposed operand would not even fit
    ref = brute_gemm(A, B)
    assert np.array_equal(oracle.gemm_u8s8s32_scalar(A, B), ref)
    assert np.array_equal(oracle.gemm_int64_numpy(A, B), ref)
    assert np.array_equal(oracle.gemm_u8s8s32_dlboost(A, B), ref)     # scalar fallback (N % 32 != 0)


def test_config1_gemm64_all_paths_agree():
    A, B = workloads.gemm_u8s8_inputs(64, 64, 64, seed=0)
    ref = oracle.gemm_int64_numpy(A, B)
    assert np.array_equal(oracle.gemm_u8s8s32_scalar(A, B), ref)
    C, path = oracle.gemm_u8s8s32_dlboost(A, B, return_path=True)
    assert np.array_equal(C, ref)
    if oracle.has_vnni():
        assert path == 2          # the vpdpbusd micro-kernel really ran


@pytest.mark.parametrize("M,K,N", [(13, 64, 32), (64, 128, 96), (200, 260, 160), (1, 4, 32)])
def test_vnni_path_vs_scalar(M, K, N):
    if not oracle.has_vnni():
        pytest.skip("host has no AVX512-VNNI")
    A, B = workloads.gemm_u8s8_inputs(M, K, N, seed=M)
    C, path = oracle.gemm_u8s8s32_dlboost(A, B, return_path=True)
    assert path == 2
    assert np.array_equal(C, oracle.gemm_u8s8s32_scalar(A, B))
    assert np.array_equal(oracle.PackedB(B).matmul(A), C)


def test_int_extremes_closed_form():
    """255 * -128 * K is the most negative sum; at K = 8192 it is -267386880 and fits int32."""
    K = 8192
    A = np.full((2, K), 255, np.uint8)
    for bv, expect in ((-128, -267386880), (127, 255 * 127 * K)):
        B = np.full((32, K), bv, np.int8)
        for C in (oracle.gemm_u8s8s32_scalar(A, B), oracle.gemm_u8s8s32_dlboost(A, B)):
            assert C.dtype == np.int32 and np.all(C == expect)
    # unsigned A: 200 must count as +200, not as int8 -56
    A = np.full((1, 4), 200, np.uint8)
    B = np.ones((32, 4), np.int8)
    assert np.all(oracle.gemm_u8s8s32_dlboost(A, B) == 800)


def test_int_bmm_is_per_batch_gemm():
    rng = np.random.default_rng(3)
    A = rng.integers(0, 256, (3, 6, 8), dtype=np.uint8)
    B = rng.integers(-128, 128, (3, 5, 8), dtype=np.int8)
    C = oracle.bmm_u8s8s32_scalar(A, B)
    for b in range(3):
        assert np.array_equal(C[b], brute_gemm(A[b], B[b]))


def test_f32_gemm_and_bmm_against_float64():
    A, B = workloads.gemm_f16_inputs(33, 72, 17, seed=2)
    ref = oracle.gemm_f64_numpy(A, B)
    got = oracle.gemm_f32(A, B)
    assert got.shape == (33, 17)
    assert np.abs(got - ref).max() <= 1e-6 * np.abs(ref).max()
    Q, Kt = workloads.bmm_qk_inputs(3, 10, 16, 12)
    assert np.abs(oracle.bmm_f32(Q, Kt) - oracle.bmm_f64_numpy(Q, Kt)).max() < 1e-5
    # identity B returns A
    eye = np.eye(72, dtype=np.float16)
    assert np.array_equal(oracle.gemm_f32(A, eye), A.astype(np.float32))


CONV = [(2, 9, 11, 8, 6, 3, 3, 1, 1, 1), (1, 8, 8, 4, 5, 1, 1, 1, 0, 1), (1, 13, 12, 3, 4, 3, 3, 2, 1, 1),
        (2, 10, 10, 2, 3, 3, 3, 1, 2, 2), (1, 7, 9, 4, 2, 5, 3, 1, 0, 1), (1, 12, 12, 2, 2, 3, 3, 3, 2, 2)]


@pytest.mark.parametrize("case", CONV)
def test_conv_against_torch_library_routine(case):
    N, H, W, CI, CO, KH, KW, s, p, d = case
    X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=sum(case))
    got = oracle.conv2d_nhwc_f32(X, Wt, s, p, d)
    x = torch.from_numpy(X.astype(np.float64)).permute(0, 3, 1, 2)            # NHWC -> NCHW
    w = torch.from_numpy(Wt.astype(np.float64)).permute(0, 3, 1, 2)           # KRSC -> KCRS
    ref = torch.nn.functional.conv2d(x, w, stride=s, padding=p, dilation=d).permute(0, 2, 3, 1).numpy()
    assert got.shape == ref.shape                                              # output-size formula
    assert got.shape[1:3] == workloads.conv_out_hw(H, W, KH, KW, s, p, d)
    assert np.abs(got - ref).max() <= 1e-5 * (np.abs(ref).max() + 1)


@pytest.mark.parametrize("case", [(1, 9, 12, 4, 3, 3, 2, (2, 1), (1, 0), (1, 2)), (2, 1, 17, 8, 5, 1, 3, (1, 2), (0, 2), (1, 1)),
                                  (1, 10, 7, 2, 2, 2, 3, (1, 1), (0, 1), (3, 1))])
def test_conv_height_and_width_parameters_differ(case):
    """stride/padding/dilation given as (height, width) pairs, fp32 and integer forms, against torch."""
    N, H, W, CI, CO, KH, KW, s, p, d = case
    X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=3)
    x = torch.from_numpy(X.astype(np.float64)).permute(0, 3, 1, 2)
    w = torch.from_numpy(Wt.astype(np.float64)).permute(0, 3, 1, 2)
    ref = torch.nn.functional.conv2d(x, w, stride=s, padding=p, dilation=d).permute(0, 2, 3, 1).numpy()
    got = oracle.conv2d_nhwc_f32(X, Wt, s, p, d)
    assert got.shape == ref.shape and np.abs(got - ref).max() <= 1e-5 * (np.abs(ref).max() + 1)
    Xi, Wi = workloads.conv2d_u8s8_inputs(N, H, W, CI, CO, KH, KW, seed=4)
    xi = torch.from_numpy(Xi.astype(np.float64)).permute(0, 3, 1, 2)
    wi = torch.from_numpy(Wi.astype(np.float64)).permute(0, 3, 1, 2)
    refi = torch.nn.functional.conv2d(xi, wi, stride=s, padding=p, dilation=d).permute(0, 2, 3, 1).numpy()
    assert np.array_equal(oracle.conv2d_nhwc_u8s8s32(Xi, Wi, s, p, d), refi.astype(np.int64))


def test_conv_1x1_reduces_to_gemm():
    X, Wt = workloads.conv2d_inputs(2, 5, 6, 8, 7, 1, 1, seed=9)
    got = oracle.conv2d_nhwc_f32(X, Wt)
    ref = oracle.gemm_f32(X.reshape(-1, 8), Wt.reshape(7, 8)).reshape(2, 5, 6, 7)
    assert np.array_equal(got, ref)


def brute_conv(X, Wt, s, p, d):
    N, H, W, CI = X.shape
    CO, KH, KW, _ = Wt.shape
    HO, WO = workloads.conv_out_hw(H, W, KH, KW, s, p, d)
    out = np.zeros((N, HO, WO, CO), np.int64)
    for n in range(N):
        for y in range(HO):
            for x in range(WO):
                for f in range(CO):
                    acc = 0
                    for ry in range(KH):
                        for rx in range(KW):
                            iy, ix = y * s + ry * d - p, x * s + rx * d - p
                            if 0 <= iy < H and 0 <= ix < W:
                                for c in range(CI):
                                    acc += int(X[n, iy, ix, c]) * int(Wt[f, ry, rx, c])
                    out[n, y, x, f] = acc
    return out


INT_CONV = [(1, 5, 6, 4, 3, 3, 3, 1, 1, 1), (2, 6, 5, 8, 4, 3, 2, 2, 1, 1), (1, 7, 7, 4, 2, 3, 3, 1, 2, 2),
            (1, 4, 4, 16, 5, 1, 1, 1, 0, 1)]


@pytest.mark.parametrize("case", INT_CONV)
def test_int_conv_against_brute_force_im2col_and_torch(case):
    N, H, W, CI, CO, KH, KW, s, p, d = case
    X, Wt = workloads.conv2d_u8s8_inputs(N, H, W, CI, CO, KH, KW, seed=sum(case))
    got = oracle.conv2d_nhwc_u8s8s32(X, Wt, s, p, d)
    assert got.dtype == np.int32
    assert np.array_equal(got, brute_conv(X, Wt, s, p, d))                    # python loops
    assert np.array_equal(got, oracle.conv2d_im2col_int64_numpy(X, Wt, s, p, d))   # explicit im2col matrix, int64
    x = torch.from_numpy(X.astype(np.float64)).permute(0, 3, 1, 2)
    w = torch.from_numpy(Wt.astype(np.float64)).permute(0, 3, 1, 2)
    ref = torch.nn.functional.conv2d(x, w, stride=s, padding=p, dilation=d).permute(0, 2, 3, 1).numpy()
    assert np.array_equal(got, ref.astype(np.int64))                           # library routine, exact in float64


def test_int_conv_unsigned_input_signed_filter_and_extremes():
    # 255 * -128 over every tap: interior pixels reach KH*KW*CI*255*-128, corners see only 4 of the 9 taps
    X = np.full((1, 5, 5, 16), 255, np.uint8)
    Wt = np.full((2, 3, 3, 16), -128, np.int8)
    got = oracle.conv2d_nhwc_u8s8s32(X, Wt, 1, 1, 1)
    assert got[0, 2, 2, 0] == 9 * 16 * 255 * -128 and got[0, 0, 0, 1] == 4 * 16 * 255 * -128
    # the input is unsigned: 200 must not be read as -56
    X = np.full((1, 1, 1, 4), 200, np.uint8)
    Wt = np.ones((1, 1, 1, 4), np.int8)
    assert oracle.conv2d_nhwc_u8s8s32(X, Wt)[0, 0, 0, 0] == 800


@pytest.mark.parametrize("cb", [32, 48, 64])
def test_int_conv_blocked_operands_equal_krsc(cb):
    """The reference's blocked filter (CO/cb,KH,KW,CI/4,cb,4) and 5-d output against the KRSC/NHWC form."""
    CO, CI = 2 * cb, 8
    X, Wt = workloads.conv2d_u8s8_inputs(1, 6, 7, CI, CO, 3, 3, seed=cb)
    Wb = oracle.pack_filter_blocked(Wt, cb)
    assert Wb.shape == (2, 3, 3, 2, cb, 4)
    # the packing itself, element by element: Wb[oc, r, s, ic, ob, ib] = Wt[oc*cb+ob, r, s, ic*4+ib]
    rng = np.random.default_rng(1)
    for _ in range(50):
        oc, r, s_, ic, ob, ib = (int(rng.integers(0, n)) for n in Wb.shape)
        assert Wb[oc, r, s_, ic, ob, ib] == Wt[oc * cb + ob, r, s_, ic * 4 + ib]
    assert np.array_equal(oracle.unpack_filter_blocked(Wb), Wt)
    got = oracle.conv2d_nhwc_u8s8s32_blocked(X, Wb, 2, 1, 1)
    assert got.shape == (1, 3, 4, 2, cb)
    assert np.array_equal(got.reshape(1, 3, 4, CO), oracle.conv2d_nhwc_u8s8s32(X, Wt, 2, 1, 1))


def test_workload_generators_are_seeded_and_shaped():
    A1, B1 = workloads.gemm_u8s8_inputs(64, 64, 64, seed=0)
    A2, B2 = workloads.gemm_u8s8_inputs(64, 64, 64, seed=0)
    assert np.array_equal(A1, A2) and np.array_equal(B1, B2)
    assert A1.dtype == np.uint8 and B1.dtype == np.int8 and A1.max() > 200 and B1.min() < -100
    P, Vt = workloads.bmm_pv_inputs(2, 8, 16, 4)
    assert np.abs(P.astype(np.float32).sum(-1) - 1).max() < 1e-2
    X, _ = workloads.conv2d_inputs(1, 8, 8, 8, 8, 3, 3)
    assert 0.3 < (X == 0).mean() < 0.7
    assert workloads.gemm_work(8192, 8192, 8192, 1, 4) == (2 * 8192 ** 3, 402653184)
    assert workloads.conv_work(32, 56, 56, 64, 64, 3, 3, 1, 1, 1) == (7398752256, 25763840)


# ---------------------------------------------------------------- operators built on a pre-stage + product
def _rand(shape, seed, scale=1.0):
    return (np.random.default_rng(seed).normal(0, scale, shape)).astype(np.float16)


def test_gemv_scan_mean_var_against_numpy_routines():
    A, b = _rand((7, 24), 1), _rand((1, 24), 2)
    g = oracle.gemv_ref(A, b)
    assert g.shape == (7, 8) and np.allclose(g[:, 0], A.astype(np.float64) @ b.astype(np.float64)[0]) and not g[:, 1:].any()
    s = oracle.scan_ref(A, 24)
    excl = np.cumsum(A.astype(np.float64), axis=1) - A.astype(np.float64)           # exclusive prefix sum
    assert np.allclose(s, excl)
    Ai = np.random.default_rng(3).integers(0, 256, (5, 32), dtype=np.uint8)
    assert np.array_equal(oracle.scan_ref(Ai, 32), np.cumsum(Ai.astype(np.int64), 1) - Ai)
    In = _rand((3, 5, 4, 6), 4)
    m = oracle.mean_ref(In)
    assert m.shape == (5, 8) and not m[:, 1:].any()
    assert np.allclose(m[:, 0], In.astype(np.float64).mean(axis=(0, 2, 3)), rtol=1e-3)   # 1/72 rounded to fp16
    Mean = np.broadcast_to(In.astype(np.float64).mean(axis=(0, 2, 3), keepdims=True), In.shape).astype(np.float16)
    v = oracle.var_ref(In, Mean)
    assert np.allclose(v[:, 0], In.astype(np.float64).var(axis=(0, 2, 3)), rtol=2e-2)


@pytest.mark.parametrize("s,p,d", [(1, 1, 1), (2, 0, 1), (1, 2, 2), (3, 1, 2)])
def test_conv1d_layouts_against_torch(s, p, d):
    X, F = _rand((2, 19, 6), 5), _rand((3, 6, 4), 6)                                  # NWC, (K,CI,CO)
    ref = torch.nn.functional.conv1d(torch.from_numpy(X.astype(np.float64)).permute(0, 2, 1),
                                     torch.from_numpy(F.astype(np.float64)).permute(2, 1, 0), stride=s, padding=p, dilation=d)
    got = oracle.conv1d_nwc_ref(X, F, s, p, d)
    assert np.allclose(got, ref.permute(0, 2, 1).numpy())
    got2 = oracle.conv1d_ncw_ref(X.transpose(0, 2, 1), F.transpose(2, 1, 0), s, p, d)
    assert np.allclose(got2, ref.numpy())


@pytest.mark.parametrize("s,p,d", [(1, 1, 1), ((2, 1), (0, 2), 1), (1, 2, 2)])
def test_conv2d_nchw_and_dil_against_torch(s, p, d):
    X, F = _rand((2, 3, 9, 8), 7), _rand((5, 3, 3, 3), 8)
    ref = torch.nn.functional.conv2d(torch.from_numpy(X.astype(np.float64)), torch.from_numpy(F.astype(np.float64)),
                                     stride=s, padding=p, dilation=d).numpy()
    assert np.allclose(oracle.conv2d_nchw_ref(X, F, s, p, d), ref)
    got = oracle.dil_nhwc_ref(X.transpose(0, 2, 3, 1), F.transpose(2, 3, 1, 0), s, p, d)
    assert np.allclose(got, ref.transpose(0, 2, 3, 1))


@pytest.mark.parametrize("s,p,d", [(1, 1, 1), ((2, 1, 1), (1, 0, 1), 1), (1, (0, 2, 1), (1, 2, 1))])
def test_conv3d_layouts_against_torch(s, p, d):
    X, F = _rand((2, 4, 6, 7, 5), 9), _rand((6, 4, 3, 3, 2), 10)                     # NCDHW, (CO,CI,KD,KH,KW)
    ref = torch.nn.functional.conv3d(torch.from_numpy(X.astype(np.float64)), torch.from_numpy(F.astype(np.float64)),
                                     stride=s, padding=p, dilation=d).numpy()
    assert np.allclose(oracle.conv3d_ncdhw_ref(X, F, s, p, d), ref)
    got = oracle.conv3d_ndhwc_ref(X.transpose(0, 2, 3, 4, 1), F.transpose(2, 3, 4, 1, 0), s, p, d)
    assert np.allclose(got, ref.transpose(0, 2, 3, 4, 1))


@pytest.mark.parametrize("s,p,d,op", [(1, 0, 1, 0), (2, 1, 1, 1), (2, 1, 1, 0), (3, 2, 2, 1), (1, 1, 2, 0)])
def test_conv2d_transposed_against_torch(s, p, d, op):
    """The declaration (expand, pad, unflipped stride-1 correlation) is a transposed convolution whose torch weight
    is the filter flipped in both window axes with the channel axes swapped."""
    X, F = _rand((2, 4, 5, 6), 11), _rand((3, 4, 3, 4), 12)                           # (N,CI,H,W), (CO,CI,KH,KW)
    w = torch.from_numpy(F.astype(np.float64)).flip(2, 3).permute(1, 0, 2, 3)        # (CI,CO,KH,KW)
    ref = torch.nn.functional.conv_transpose2d(torch.from_numpy(X.astype(np.float64)), w, stride=s, padding=p,
                                               output_padding=op, dilation=d).numpy()
    got = oracle.conv2d_transposed_nchw_ref(X, F, s, p, d, op)
    assert got.shape == ref.shape and np.allclose(got, ref)


@pytest.mark.parametrize("s,p,mult", [(1, 1, 1), (2, 1, 2), (1, 0, 3)])
def test_depthwise_conv_against_torch_grouped_conv(s, p, mult):
    X, F = _rand((2, 5, 9, 8), 13), _rand((5 * mult, 3, 3), 14)
    ref = torch.nn.functional.conv2d(torch.from_numpy(X.astype(np.float64)), torch.from_numpy(F.astype(np.float64)).unsqueeze(1),
                                     stride=s, padding=p, groups=5).numpy()                 # (N, C*mult, HO, WO)
    got = oracle.depthwise_conv2d_ref(X, F, s, p)
    assert got.shape[:3] == (2, 5, 8) and not got[:, :, mult:].any()
    assert np.allclose(got[:, :, :mult].reshape(2, 5 * mult, *got.shape[3:]), ref)
