"""GPU parity: every shipped template instance against the CPU oracle, through the C ABI.

Integer results must be bit-exact.  fp16 results (fp32 accumulate, one rounding to fp16) must be
within REL_TOL of the fp32 host reference, measured as max|err| / max|ref| per tensor, plus an
element-wise check with an fp16-rounding allowance.
"""
import numpy as np
import pytest
import torch

import oracle
from heron_amd import backend as B
from heron_amd import hostops, instances, workloads
from parity_checks import REL_TOL, check_f16

pytestmark = pytest.mark.gpu

_mods = {}


def mod_for(desc):
    key = desc.as_tuple()
    if key not in _mods:
        _mods[key] = B.Module(desc)
    return _mods[key]


def dev(a):
    return torch.from_numpy(a).cuda()


GEMM_SHAPES = [(64, 64, 64), (256, 256, 256), (512, 640, 384), (100, 200, 72), (8, 4096, 16), (300, 1024, 520)]


@pytest.mark.parametrize("tup", instances.PARITY_SHAPES, ids=lambda t: "x".join(map(str, t)))
def test_gemm_u8s8_bit_exact(tup, hrn):
    m = mod_for(instances.D(instances.U8, instances.GEMM, *tup))
    for i, (M, K, N) in enumerate(GEMM_SHAPES):
        K16 = (K + 15) // 16 * 16
        A, Bm = workloads.gemm_u8s8_inputs(M, K16, N, seed=10 + i)
        print("u8s8", tup, (M, K16, N), flush=True)
        C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
        ref = oracle.gemm_u8s8s32_dlboost(A, Bm) if N % 32 == 0 else oracle.gemm_int64_numpy(A, Bm).astype(np.int32)
        assert np.array_equal(C, ref)


@pytest.mark.parametrize("tup", instances.PARITY_SHAPES, ids=lambda t: "x".join(map(str, t)))
def test_gemm_f16_within_tolerance(tup, hrn):
    m = mod_for(instances.D(instances.F16, instances.GEMM, *tup))
    for i, (M, K, N) in enumerate(GEMM_SHAPES):
        K8 = (K + 7) // 8 * 8
        A, Bm = workloads.gemm_f16_inputs(M, K8, N, seed=20 + i, scale=1.0 if i % 2 else 0.1)
        print("f16", tup, (M, K8, N), flush=True)
        C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
        check_f16(C, oracle.gemm_f32(A, Bm))


@pytest.mark.parametrize("desc", instances.variant_descs(), ids=lambda d: "-".join(map(str, d.as_tuple())))
def test_template_variants(desc, hrn):
    """LDS-staged epilogue, one k-step per k-tile (alternating register buffers), window and im2col conv load paths."""
    m = mod_for(desc)
    if desc.op == instances.CONV and desc.conv_window:
        same = [(2, 14, 14, 64, 64, 3, 3, 1, 1, 1), (1, 9, 11, 64, 32, 3, 3, 1, 1, 1), (2, 8, 8, 64, 48, 1, 1, 1, 0, 1),
                (3, 7, 7, 128, 64, 5, 5, 1, 2, 1), (2, 56, 56, 64, 64, 3, 3, 1, 1, 1)]
        for i, case in enumerate(same):
            N, H, W, CI, CO, KH, KW, s, p, d = case
            X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=70 + i)
            print("window conv", desc.as_tuple(), case, flush=True)
            Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy()
            check_f16(Y, oracle.conv2d_nhwc_f32(X, Wt, s, p, d))
        # shapes the window path cannot serve are refused, not mis-computed
        for case in [(1, 15, 15, 64, 16, 3, 3, 2, 1, 1), (1, 12, 12, 64, 8, 3, 3, 1, 2, 2), (1, 9, 9, 64, 8, 3, 3, 1, 0, 1),
                     (1, 5, 600, 128, 16, 3, 3, 1, 1, 1)]:
            N, H, W, CI, CO, KH, KW, s, p, d = case
            X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=1)
            with pytest.raises(B.HeronRocmError):
                hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d)
        return
    if desc.op == instances.CONV:
        for i, case in enumerate(CONV_CASES[:4]):
            N, H, W, CI, CO, KH, KW, s, p, d = case
            X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=40 + i)
            print("variant conv", desc.as_tuple(), case, flush=True)
            Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy()
            check_f16(Y, oracle.conv2d_nhwc_f32(X, Wt, s, p, d))
        return
    for i, (M, K, N) in enumerate(GEMM_SHAPES + [(1024, 2048, 768)]):
        K16 = (K + 15) // 16 * 16
        print("variant", desc.as_tuple(), (M, K16, N), flush=True)
        if desc.dtype == instances.U8:
            A, Bm = workloads.gemm_u8s8_inputs(M, K16, N, seed=50 + i)
            C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
            assert np.array_equal(C, oracle.gemm_int64_numpy(A, Bm).astype(np.int32))
        else:
            A, Bm = workloads.gemm_f16_inputs(M, K16, N, seed=60 + i)
            C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
            check_f16(C, oracle.gemm_f32(A, Bm))


def test_gemm_u8s8_extremes(hrn):
    """A = 255, B = -128 reaches the most negative accumulator; B = 127 the most positive."""
    m = mod_for(instances.BEST["small"])
    M = N = 64
    for K in (64, 4096, 8192):
        A = np.full((M, K), 255, np.uint8)
        for bv in (-128, 127):
            Bm = np.full((N, K), bv, np.int8)
            C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
            assert np.all(C == 255 * bv * K)
        # identity-like B picks single columns of A
        A2, _ = workloads.gemm_u8s8_inputs(M, K, N, seed=K)
        Bm = np.zeros((N, K), np.int8)
        Bm[np.arange(N), np.arange(N)] = 1
        C = hostops.gemm(m, dev(A2), dev(Bm)).cpu().numpy()
        assert np.array_equal(C, A2[:, :N].astype(np.int32))


def test_gemm_f16_exact_cases(hrn):
    """Power-of-two scaling is exact; integer-valued inputs with small sums are exact in fp16."""
    m = mod_for(instances.BEST["small_f16"])
    rng = np.random.default_rng(7)
    A = rng.integers(-4, 5, (96, 64)).astype(np.float16)
    Bm = rng.integers(-4, 5, (80, 64)).astype(np.float16)
    C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
    ref = (A.astype(np.int64) @ Bm.astype(np.int64).T)
    assert np.array_equal(C.astype(np.int64), ref)          # |sum| <= 1024 < 2048: exact in fp16
    C4 = hostops.gemm(m, dev((A * 4).astype(np.float16)), dev(Bm)).cpu().numpy()
    assert np.array_equal(C4, C * 4)


@pytest.mark.parametrize("tup", instances.PARITY_SHAPES[:5], ids=lambda t: "x".join(map(str, t)))
def test_bmm_f16(tup, hrn):
    m = mod_for(instances.D(instances.F16, instances.GEMM, *tup))
    for (b, M, K, N) in [(3, 128, 64, 192), (5, 72, 128, 40)]:
        Q, Kt = workloads.bmm_qk_inputs(b, M, K, N, seed=b)
        print("bmm", tup, (b, M, K, N), flush=True)
        C = hostops.gemm(m, dev(Q), dev(Kt)).cpu().numpy()
        check_f16(C, oracle.bmm_f32(Q, Kt))
        # batch independence: a permuted batch gives the permuted result, bit for bit
        perm = np.roll(np.arange(b), 1)
        Cp = hostops.gemm(m, dev(Q[perm].copy()), dev(Kt[perm].copy())).cpu().numpy()
        assert np.array_equal(Cp, C[perm])
    P, Vt = workloads.bmm_pv_inputs(2, 64, 128, 64, seed=3)
    ones = np.ones((2, 8, 128), np.float16)
    R = hostops.gemm(m, dev(P), dev(ones)).cpu().numpy()     # rows of P sum to 1
    assert np.abs(R.astype(np.float32) - 1).max() < 5e-3


def test_bmm_u8s8(hrn):
    m = mod_for(instances.BEST["small"])
    rng = np.random.default_rng(11)
    A = rng.integers(0, 256, (4, 96, 80), dtype=np.uint8)
    Bm = rng.integers(-128, 128, (4, 72, 80), dtype=np.int8)
    C = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
    assert np.array_equal(C, oracle.bmm_u8s8s32_scalar(A, Bm))


CONV_CASES = [
    # N, H, W, CI, CO, KH, KW, stride, pad, dil
    (2, 14, 14, 64, 64, 3, 3, 1, 1, 1),
    (1, 9, 11, 16, 32, 3, 3, 1, 1, 1),
    (2, 8, 8, 32, 48, 1, 1, 1, 0, 1),
    (1, 15, 15, 8, 16, 3, 3, 2, 1, 1),
    (1, 12, 12, 24, 8, 3, 3, 1, 2, 2),
    (3, 7, 7, 128, 64, 5, 5, 1, 2, 1),
]


def _conv_tuples():
    return [d.as_tuple()[2:10] for d in instances.parity_descs() if d.op == instances.CONV]


@pytest.mark.parametrize("tup", _conv_tuples(), ids=lambda t: "x".join(map(str, t)))
def test_conv2d_nhwc_f16(tup, hrn):
    m = mod_for(instances.D(instances.F16, instances.CONV, *tup))
    for i, (N, H, W, CI, CO, KH, KW, s, p, d) in enumerate(CONV_CASES):
        X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=30 + i)
        print("conv", tup, CONV_CASES[i], flush=True)
        Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy()
        check_f16(Y, oracle.conv2d_nhwc_f32(X, Wt, s, p, d))


INT8_CONV_CASES = [
    # N, H, W, CI, CO, KH, KW, stride, pad, dil      (CI a multiple of 16: whole 16-byte channel chunks)
    (2, 14, 14, 64, 64, 3, 3, 1, 1, 1),
    (1, 9, 11, 16, 32, 3, 3, 1, 1, 1),
    (2, 8, 8, 32, 48, 1, 1, 1, 0, 1),
    (1, 15, 15, 16, 16, 3, 3, 2, 1, 1),
    (1, 12, 12, 48, 8, 3, 3, 1, 2, 2),
    (3, 7, 7, 128, 64, 5, 5, 1, 2, 1),
]


def test_caller_supplied_column_sums(hrn):
    """colsum instances: hrn_colsum_s8 equals the sum over K (int64 numpy); the product with the sums handed over
    explicitly, with the sums made on the spot, and of the in-kernel instance are all the oracle's, bit for bit -
    GEMM, batched, ragged; a launch through the C ABI without the sums is refused, not mis-computed."""
    import ctypes
    rng = np.random.default_rng(21)
    Bm = rng.integers(-128, 128, (3, 200, 272), dtype=np.int8)
    Bm[0, 0, :] = -128
    Bm[1, 5, :] = 127
    got = hostops.column_sums(dev(Bm)).cpu().numpy()
    assert got.dtype == np.int32 and np.array_equal(got, Bm.astype(np.int64).sum(axis=2))
    Wt = rng.integers(-128, 128, (48, 3, 3, 32), dtype=np.int8)
    assert np.array_equal(hostops.column_sums(dev(Wt)).cpu().numpy(), Wt.astype(np.int64).sum(axis=(1, 2, 3)))
    m = mod_for(instances.D(instances.U8, instances.GEMM, 64, 128, 256, 1, 2, 16, 2, 1, epi=1, colsum=1))
    for i, (M, K, N) in enumerate([(64, 64, 64), (300, 1040, 520), (100, 208, 72)]):
        A, B2 = workloads.gemm_u8s8_inputs(M, K, N, seed=400 + i)
        ref = oracle.gemm_int64_numpy(A, B2).astype(np.int32)
        dB = dev(B2)
        assert np.array_equal(hostops.gemm(m, dev(A), dB, bsum=hostops.column_sums(dB)).cpu().numpy(), ref)
        assert np.array_equal(hostops.gemm(m, dev(A), dB).cpu().numpy(), ref)
    A = rng.integers(0, 256, (3, 96, 272), dtype=np.uint8)
    assert np.array_equal(hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy(), oracle.bmm_u8s8s32_scalar(A, Bm))
    # extremes: 255 x -128 over all of K with the sums supplied
    A = np.full((64, 8192), 255, np.uint8)
    B3 = np.full((64, 8192), -128, np.int8)
    assert int(hostops.gemm(m, dev(A), dev(B3)).cpu().numpy()[0, 0]) == -267386880
    # the raw entry point refuses a colsum instance without the sums
    A, B2 = workloads.gemm_u8s8_inputs(64, 64, 64, seed=1)
    dA, dB, out = dev(A), dev(B2), torch.empty((64, 64), dtype=torch.int32, device="cuda")
    p = B.gemm_problem(1, 64, 64, 64)
    rc = B.lib().hrn_launch_gemm_u8s8(m._h, ctypes.byref(p), dA.data_ptr(), dB.data_ptr(), out.data_ptr(), 0)
    assert rc == B.HRN_E_BADPARAM and b"bsum" in B.lib().hrn_last_error()
    # and fp16 instances have no such option
    assert not B.check_desc(instances.D(instances.F16, instances.GEMM, 128, 128, 128, 2, 2, 32, 2, 1, colsum=1))


@pytest.mark.parametrize("desc", instances.int8_conv_descs(), ids=lambda d: "-".join(map(str, d.as_tuple())))
def test_conv2d_nhwc_u8s8_bit_exact(desc, hrn):
    m = mod_for(desc)
    ran = 0
    for i, case in enumerate(INT8_CONV_CASES):
        N, H, W, CI, CO, KH, KW, s, p, d = case
        X, Wt = workloads.conv2d_u8s8_inputs(N, H, W, CI, CO, KH, KW, seed=90 + i)
        print("int8 conv", desc.as_tuple(), case, flush=True)
        if desc.conv_window and (s != 1 or d != 1 or 2 * p != (KH - 1) or CI % desc.bkb):
            with pytest.raises(B.HeronRocmError):
                hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d)
            continue
        Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy()
        assert Y.dtype == np.int32 and np.array_equal(Y, oracle.conv2d_nhwc_u8s8s32(X, Wt, s, p, d))
        ran += 1
    assert ran >= 1


def test_conv2d_u8s8_extremes_and_blocked_filter(hrn):
    """255 x -128 on every tap (largest magnitude the int32 sum sees) and weights handed over in the
    blocked (CO/b,KH,KW,CI/4,b,4) order of the x86 operator, reordered once on the device."""
    m = mod_for(instances.int8_conv_descs()[1])
    X = np.full((1, 6, 6, 64), 255, np.uint8)
    Wt = np.full((64, 3, 3, 64), -128, np.int8)
    Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), 1, 1, 1).cpu().numpy()
    assert Y[0, 2, 2, 0] == 9 * 64 * 255 * -128 and Y[0, 0, 0, 63] == 4 * 64 * 255 * -128
    assert np.array_equal(Y, oracle.conv2d_nhwc_u8s8s32(X, Wt, 1, 1, 1))
    X, Wt = workloads.conv2d_u8s8_inputs(2, 9, 9, 32, 96, 3, 3, seed=8)
    for cb in (32, 48):
        Wb = oracle.pack_filter_blocked(Wt, cb)
        Wk = hostops.unpack_filter_blocked(dev(Wb))
        assert np.array_equal(Wk.cpu().numpy(), Wt)
        Y = hostops.conv2d_nhwc(m, dev(X), Wk, 2, 1, 1).cpu().numpy()
        ref = oracle.conv2d_nhwc_u8s8s32_blocked(X, Wb, 2, 1, 1)              # (N,HO,WO,CO/cb,cb)
        assert np.array_equal(Y.reshape(ref.shape), ref)


PERSIST_GEMM_SHAPES = [(4096, 64, 4096), (1000, 80, 2056), (2048, 528, 512), (96, 4096, 40)]     # (M, K, N), N*out_bytes % 16 == 0


@pytest.mark.parametrize("grid", ["", "8", "40"], ids=["device-filling", "8-workgroups", "40-workgroups"])
@pytest.mark.parametrize("desc", instances.persistent_descs(), ids=lambda d: "-".join(map(str, d.as_tuple())))
def test_persistent_tile_stream(desc, grid, hrn, monkeypatch):
    """Persistent instances: every workgroup walks several output tiles and fetches the next tile's operands while the
    current result is stored.  Few workgroups (8, 40) force many tiles per workgroup, also with short K streams
    (one or two k-tiles per output tile, i.e. several epilogues inside the fetch window)."""
    if grid:
        monkeypatch.setenv("HRN_PERSIST_GRID", grid)
    else:
        monkeypatch.delenv("HRN_PERSIST_GRID", raising=False)
    m = mod_for(desc)
    f16 = desc.dtype == instances.F16
    if desc.op == instances.CONV:
        cases = [(2, 14, 14, 64, 64, 3, 3, 1, 1, 1), (3, 17, 15, 32, 48, 3, 3, 2, 1, 1), (1, 12, 12, 16, 8, 1, 1, 1, 0, 1),
                 (8, 28, 28, 64, 64, 3, 3, 1, 1, 1)]
        for i, case in enumerate(cases):
            N, H, W, CI, CO, KH, KW, s, p, d = case
            print("persistent conv", desc.as_tuple(), grid, case, flush=True)
            if f16:
                X, Wt = workloads.conv2d_inputs(N, H, W, CI, CO, KH, KW, seed=110 + i)
                check_f16(hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy(), oracle.conv2d_nhwc_f32(X, Wt, s, p, d))
            else:
                X, Wt = workloads.conv2d_u8s8_inputs(N, H, W, CI, CO, KH, KW, seed=110 + i)
                assert np.array_equal(hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, d).cpu().numpy(),
                                      oracle.conv2d_nhwc_u8s8s32(X, Wt, s, p, d))
        return
    for i, (M, K, N) in enumerate(PERSIST_GEMM_SHAPES):
        print("persistent gemm", desc.as_tuple(), grid, (M, K, N), flush=True)
        if f16:
            A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=120 + i)
            check_f16(hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy(), oracle.gemm_f32(A, Bm))
        else:
            A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=120 + i)
            assert np.array_equal(hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy(), oracle.gemm_int64_numpy(A, Bm))
    # batched, and bit-identical to the one-tile-per-workgroup instance of the same tile (same summation order)
    t = desc.as_tuple()
    plain = mod_for(instances.D(desc.dtype, desc.op, *t[2:10], epi=1))
    if f16:
        A, Bm = workloads.bmm_qk_inputs(24, 512, 64, 512, seed=7)
    else:
        rng = np.random.default_rng(3)
        A = rng.integers(0, 256, (24, 512, 64), dtype=np.uint8)
        Bm = rng.integers(-128, 128, (24, 512, 64), dtype=np.int8)
    C1 = hostops.gemm(m, dev(A), dev(Bm)).cpu().numpy()
    C0 = hostops.gemm(plain, dev(A), dev(Bm)).cpu().numpy()
    assert np.array_equal(C1, C0)


def test_persistent_rejects_partial_chunks(hrn):
    m = mod_for(instances.persistent_descs()[0])
    A, Bm = workloads.gemm_f16_inputs(64, 64, 36, seed=1)              # N*2 is not a multiple of 16
    with pytest.raises(B.HeronRocmError):
        hostops.gemm(m, dev(A), dev(Bm))


@pytest.mark.parametrize("desc", instances.splitk_descs(), ids=lambda d: "-".join(map(str, d.as_tuple())))
def test_split_k(desc, hrn):
    """K cut into slices that run as separate workgroups: partial sums + the reduction pass give the one-pass result
    (uint8 bit-exact, fp16 within 1e-2) for slice counts that divide the k-tiles, that do not, that exceed them, and 1."""
    m = mod_for(desc)
    f16 = desc.dtype == instances.F16
    if desc.op == instances.CONV:
        cases = [(16, 7, 7, 512, 64, 3, 3, 1, 1, 1), (2, 15, 15, 64, 48, 3, 3, 2, 1, 1), (1, 9, 9, 32, 16, 5, 5, 1, 2, 2)]
        for i, case in enumerate(cases):
            N, H, W, CI, CO, KH, KW, st, pd, dl = case
            gen = workloads.conv2d_inputs if f16 else workloads.conv2d_u8s8_inputs
            X, Wt = gen(N, H, W, CI, CO, KH, KW, seed=300 + i)
            ref = oracle.conv2d_nhwc_f32(X, Wt, st, pd, dl) if f16 else oracle.conv2d_nhwc_u8s8s32(X, Wt, st, pd, dl)
            for split in (1, 2, 3, 8, 64):
                print("split-k conv", desc.as_tuple(), case, split, flush=True)
                Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), st, pd, dl, split_k=split).cpu().numpy()
                if f16:
                    check_f16(Y, ref)
                else:
                    assert np.array_equal(Y, ref)
        return
    for i, (M, K, N) in enumerate([(100, 4096, 72), (784, 4608, 256), (64, 64, 64), (130, 1040, 36)]):
        if f16:
            A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=310 + i)
            ref = oracle.gemm_f32(A, Bm)
        else:
            A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=310 + i)
            ref = oracle.gemm_int64_numpy(A, Bm).astype(np.int32)
        for split in (1, 2, 5, 16, 1000):
            print("split-k gemm", desc.as_tuple(), (M, K, N), split, flush=True)
            C = hostops.gemm(m, dev(A), dev(Bm), split_k=split).cpu().numpy()
            if f16:
                check_f16(C, ref)
            else:
                assert np.array_equal(C, ref)
    # batched: every batch entry has its own slices
    if f16:
        A = np.stack([workloads.gemm_f16_inputs(96, 2048, 40, seed=330 + b)[0] for b in range(3)])
        Bm = np.stack([workloads.gemm_f16_inputs(96, 2048, 40, seed=330 + b)[1] for b in range(3)])
        C = hostops.gemm(m, dev(A), dev(Bm), split_k=4).cpu().numpy()
        for b in range(3):
            check_f16(C[b], oracle.gemm_f32(A[b], Bm[b]))


def test_split_k_error_paths(hrn):
    """A split-K instance without (or with too small a) workspace, and a slice count on an instance built without
    split_k, are refused."""
    d = instances.splitk_descs()[0]
    m = mod_for(d)
    A, Bm = workloads.gemm_f16_inputs(64, 1024, 64, seed=1)
    a, b = dev(A), dev(Bm)
    c = torch.empty((64, 64), dtype=torch.float16, device="cuda")
    L = B.lib()
    p = B.gemm_problem(1, 64, 64, 1024, 8, split_k=4)
    need = B.splitk_workspace_bytes(d, p)
    assert need == 4 * 64 * 64 * 4
    import ctypes
    assert L.hrn_launch_gemm_f16(m._h, ctypes.byref(p), a.data_ptr(), b.data_ptr(), c.data_ptr(), 0) == B.HRN_E_BADPARAM
    assert b"workspace" in L.hrn_last_error()
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    p.workspace, p.workspace_bytes = ws.data_ptr(), need - 16
    assert L.hrn_launch_gemm_f16(m._h, ctypes.byref(p), a.data_ptr(), b.data_ptr(), c.data_ptr(), 0) == B.HRN_E_BADPARAM
    assert b"too small" in L.hrn_last_error()
    p.workspace_bytes = need
    assert L.hrn_launch_gemm_f16(m._h, ctypes.byref(p), a.data_ptr(), b.data_ptr(), c.data_ptr(), 0) == B.HRN_OK
    torch.cuda.synchronize()
    check_f16(c.cpu().numpy(), oracle.gemm_f32(A, Bm))
    plain = mod_for(instances.BEST["small_f16"])
    with pytest.raises(B.HeronRocmError):
        hostops.gemm(plain, a, b, split_k=2)
    p0 = B.gemm_problem(1, 64, 64, 1024, 8)
    assert B.splitk_workspace_bytes(instances.BEST["small_f16"], p0) == 0


def test_conv_1x1_is_gemm(hrn):
    """A 1x1 convolution is the GEMM of the flattened pixels: both templates must agree bit for bit."""
    tup = instances.PARITY_SHAPES[2]
    mc = mod_for(instances.D(instances.F16, instances.CONV, *tup))
    mg = mod_for(instances.D(instances.F16, instances.GEMM, *tup))
    X, Wt = workloads.conv2d_inputs(2, 8, 8, 64, 64, 1, 1, seed=5)
    Y = hostops.conv2d_nhwc(mc, dev(X), dev(Wt)).cpu().numpy()
    G = hostops.gemm(mg, dev(X.reshape(-1, 64)), dev(Wt.reshape(64, 64))).cpu().numpy()
    assert np.array_equal(Y.reshape(-1, 64), G)


def test_error_paths(hrn):
    """Bad descriptors and problems come back as error codes, not as launches."""
    bad = instances.D(instances.F16, instances.GEMM, 256, 256, 128, 2, 2, 32, 3, 2)   # 192 KiB of LDS
    assert not B.check_desc(bad)
    with pytest.raises(B.HeronRocmError):
        B.Module(bad)
    m = mod_for(instances.BEST["small_f16"])
    A = torch.zeros((64, 60), dtype=torch.float16, device="cuda")       # K*2 not a multiple of 16
    with pytest.raises(B.HeronRocmError):
        hostops.gemm(m, A, A)
    mu = mod_for(instances.BEST["small"])
    with pytest.raises(ValueError):
        hostops.gemm(mu, A, A)                                           # wrong dtype for the module


def test_hip_measurer_tunes_gemm64(hrn, tmp_path):
    """The reference's quick-start case end to end on the GPU: 64^3 u8s8 GEMM, CGA, HIP builder + measurement
    server, results verified against a host reference inside the measurer (Task.set_verify_func)."""
    from heron_amd.config import Config
    from heron_amd.environment import Env
    from heron_amd.ops.rocm import getOpFromName
    from heron_amd import runner as R
    cfg = Config()
    cfg.codegen_type, cfg.target_name, cfg.get_op = 'GPU_MFMA', 'rocm', getOpFromName
    cfg.out_name = str(tmp_path / "OPS")
    cfg.opt_method, cfg.max_trials, cfg.measure_time_per_round = 'CGA', 24, 8
    cfg.pop_num, cfg.select_num, cfg.iter_walks, cfg.parallel_num = 24, 12, 2, 2
    cfg.in_dtype, cfg.out_dtype = 'int8', 'int32'
    runner = R.LocalRunner(number=2, repeat=3, min_repeat_ms=0, timeout=60)
    builder = R.LocalBuilder(timeout=60, n_parallel=4)
    try:
        env = Env(R.measure_option(builder, runner), cfg)
        task = env.createTask("G1", getOpFromName("gemm"), [64, 64, 64, 'int8', 'int32'], 'rocm')
        assert env.build_kwargs['check_gpu']['lds_bytes_per_wg'] == 163840

        def ref(args):
            A, Bm = workloads.gemm_u8s8_inputs(64, 64, 64, seed=0)
            return [A, Bm], oracle.gemm_int64_numpy(A, Bm)
        task.set_verify_func(ref, rtol=1e-6)
        env.tune("G1")
        import json
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / "G1" / "records.txt")]
        assert len(rows) >= 16 and all(r["perf"] > 0 for r in rows)         # every kernel ran and verified
        best = max(r["perf"] for r in rows)
        assert np.exp(-best) < 50e-6
        s, args = task.apply_best(str(tmp_path / "OPS" / "G1" / "records.txt"))
        assert runner.time_instance(s, args, number=2, repeat=2, min_repeat_ms=1) > 0
        # a wrong expected output must be reported as error 100 -> perf 0
        task.ref_output = task.ref_output + 1
        from heron_amd.sample import Sample
        smp = Sample(task)
        _, point = smp.knob_manager.randSample({})
        smp.point, smp.stmt_code = point, "wrong_" + "_".join(map(str, point))
        env.runner.measure_batch = R.create_measure_batch(task, env.runner.measure_option)
        env.evalSamples([smp])
        assert smp.perf == 0.0 and not smp.valid
    finally:
        runner.close()
        builder.close()


def test_device_info_and_timing(hrn):
    info = B.device_info(0)
    assert info["arch"].startswith("gfx950") and info["wave_size"] == 64 and info["cu_count"] > 0
    m = mod_for(instances.BEST["small_f16"])
    A, Bm = workloads.gemm_f16_inputs(256, 256, 256)
    a, b = dev(A), dev(Bm)
    c = torch.empty((256, 256), dtype=torch.float16, device="cuda")
    costs = m.time(B.gemm_problem(1, 256, 256, 256), a.data_ptr(), b.data_ptr(), c.data_ptr(), number=3, repeat=4,
                   min_repeat_ms=1.0)
    assert len(costs) == 4 and all(0 < x < 1e-2 for x in costs)
    check_f16(c.cpu().numpy(), oracle.gemm_f32(A, Bm))


def test_cold_cache_timing(hrn):
    """Launches timed after a cache flush: the 4 MiB-operand GEMM that lives in L2/MALL when repeated takes longer
    from HBM, and the result is still correct."""
    from heron_amd import tuned
    m = mod_for(tuned.load("gemm_f16_4096").desc)
    A, Bm = workloads.gemm_f16_inputs(2048, 1024, 2048, seed=4)
    a, b = dev(A), dev(Bm)
    c = torch.empty((2048, 2048), dtype=torch.float16, device="cuda")
    flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    p = B.gemm_problem(1, 2048, 2048, 1024, 4)
    warm = sorted(m.time(p, a.data_ptr(), b.data_ptr(), c.data_ptr(), number=20, repeat=5))[2]
    cold = sorted(m.time_cold(p, a.data_ptr(), b.data_ptr(), c.data_ptr(), flush.data_ptr(), flush.numel(), repeat=5))[2]
    print("warm %.2f us, cold %.2f us" % (warm * 1e6, cold * 1e6), flush=True)
    assert warm > 0 and 0.8 * warm < cold < 100 * warm          # cold is slower; the margin only absorbs timing noise
    check_f16(c.cpu().numpy(), oracle.gemm_f32(A, Bm))
    with pytest.raises(B.HeronRocmError):
        m.time_cold(p, a.data_ptr(), b.data_ptr(), c.data_ptr(), flush.data_ptr(), 1024, repeat=2)


def test_launches_from_several_host_threads(hrn):
    """Four host threads launch through the same library at once, each on a stream of its own: two share one module,
    two have their own.  Every result must match what the oracle gives for that thread's inputs."""
    import threading
    shared = mod_for(instances.BEST["small_f16"])
    mods = [shared, shared, mod_for(instances.BEST["small"]), mod_for(instances.D(instances.F16, instances.GEMM, *instances.PARITY_SHAPES[0]))]
    shapes = [(192, 128, 320), (130, 72, 64), (256, 144, 96), (64, 264, 200)]
    inputs, outs, errors = [], [None] * 4, []
    for i, (m, (M, K, N)) in enumerate(zip(mods, shapes)):
        gen = workloads.gemm_f16_inputs if m.desc.dtype == B.HRN_DT_F16 else workloads.gemm_u8s8_inputs
        A, Bm = gen(M, K, N, seed=70 + i)
        inputs.append((A, Bm, dev(A), dev(Bm)))
    torch.cuda.synchronize()
    start = threading.Barrier(4)

    def work(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                start.wait()
                for _ in range(50):
                    out = hostops.gemm(mods[i], inputs[i][2], inputs[i][3])
                s.synchronize()
            outs[i] = out.cpu().numpy()
        except Exception as e:       # reported by the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    assert not errors, errors
    for i, m in enumerate(mods):
        A, Bm = inputs[i][0], inputs[i][1]
        if m.desc.dtype == B.HRN_DT_F16:
            check_f16(outs[i], oracle.gemm_f32(A, Bm))
        else:
            assert np.array_equal(outs[i], oracle.gemm_int64_numpy(A, Bm).astype(np.int32))
