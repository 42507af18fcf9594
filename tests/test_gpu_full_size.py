"""The benchmarked instances at the benchmark's full sizes (the shapes `bench.py` times, same tile instance and raster).

A full CPU product of 8192^3 is out of reach for a test, so each result is pinned by
* the oracle on a random subset of rows / batch entries / images (bit-exact for uint8 x int8, rel. error <= 1e-2 for
  fp16 inputs with fp32 accumulation), and
* checksums of checksums that cover EVERY output element: sum_j C[i,j] = A[i,:] . (sum_j B[j,:]) for every row i and
  sum_i C[i,j] = (sum_i A[i,:]) . B[j,:] for every column j, exact in int64 for the integer path, within the fp16
  output rounding (2^-11 per element, accumulated as a random walk) for the floating point one.  A single wrong
  element breaks one row identity and one column identity.
"""
import numpy as np
import pytest
import torch

import oracle
from heron_amd import backend as B
from heron_amd import hostops, instances, tuned, workloads
from parity_checks import check_f16

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(a).cuda()


# benchmark workload behind each short key used below
TUNED_KEY = {"gemm_f16_4096": "gemm_f16_4096", "gemm_f16": "gemm_f16_8192", "gemm_u8s8": "gemm_u8s8_8192",
             "bmm_f16_qk": "bmm_f16_qk", "bmm_f16_pv": "bmm_f16_pv", "conv2d_f16": "conv2d_f16_resnet",
             "conv2d_u8s8": "conv2d_u8s8_resnet"}


def module(key):
    """The tuned instance the benchmark runs for this workload (best record, through Task.apply_best)."""
    inst = tuned.load(TUNED_KEY[key])
    print("tuned instance", key, inst.desc.as_tuple(), "group_m", inst.group_m, flush=True)
    return B.Module(inst.desc), inst.group_m


def check_rows_f16(C, A, Bm, rows):
    check_f16(C[rows], oracle.gemm_f32(A[rows], Bm))


def check_sums_f16(C, A, Bm):
    """Row and column checksums in float64 against the closed forms; tolerance = fp16 rounding of the outputs."""
    C64 = C.astype(np.float64)
    A64, B64 = A.astype(np.float64), Bm.astype(np.float64)
    cmax = float(np.abs(C64).max())
    M, N = C.shape
    row_ref = A64 @ B64.sum(axis=0)
    col_ref = A64.sum(axis=0) @ B64.T
    # each output carries a rounding error <= 2^-11 |C|; a sum of n of them stays within 8 sqrt(n) 2^-11 max|C|
    assert np.abs(C64.sum(axis=1) - row_ref).max() <= 8 * np.sqrt(N) * 2.0 ** -11 * cmax
    assert np.abs(C64.sum(axis=0) - col_ref).max() <= 8 * np.sqrt(M) * 2.0 ** -11 * cmax


@pytest.mark.parametrize("key,size", [("gemm_f16_4096", 4096), ("gemm_f16", 8192)])
def test_gemm_f16_full_size(key, size, hrn):
    m, gm = module(key)
    A, Bm = workloads.gemm_f16_inputs(size, size, size, seed=1)
    C = hostops.gemm(m, dev(A), dev(Bm), group_m=gm).cpu().numpy()
    rows = np.random.default_rng(0).choice(size, 48, replace=False)
    check_rows_f16(C, A, Bm, np.sort(rows))
    check_sums_f16(C, A, Bm)


def test_gemm_u8s8_full_size(hrn):
    m, gm = module("gemm_u8s8")
    A, Bm = workloads.gemm_u8s8_inputs(8192, 8192, 8192, seed=2)
    C = hostops.gemm(m, dev(A), dev(Bm), group_m=gm).cpu().numpy()
    rows = np.sort(np.random.default_rng(1).choice(8192, 64, replace=False))
    assert np.array_equal(C[rows], oracle.gemm_u8s8s32_dlboost(A[rows], Bm))
    A64, B64 = A.astype(np.int64), Bm.astype(np.int64)
    assert np.array_equal(C.sum(axis=1, dtype=np.int64), A64 @ B64.sum(axis=0))
    assert np.array_equal(C.sum(axis=0, dtype=np.int64), A64.sum(axis=0) @ B64.T)


@pytest.mark.parametrize("key,gen,shape", [("bmm_f16_qk", workloads.bmm_qk_inputs, (192, 512, 64, 512)),
                                           ("bmm_f16_pv", workloads.bmm_pv_inputs, (192, 512, 512, 64))])
def test_bmm_full_size(key, gen, shape, hrn):
    m, gm = module(key)
    A, Bm = gen(*shape)
    C = hostops.gemm(m, dev(A), dev(Bm), group_m=gm).cpu().numpy()
    for b in (0, 1, 95, 190, 191):
        ref = oracle.gemm_f32(A[b], Bm[b])
        check_f16(C[b], ref)
    # every batch entry: row checksums against the closed form
    A64, B64, C64 = A.astype(np.float64), Bm.astype(np.float64), C.astype(np.float64)
    row_ref = np.einsum("bik,bk->bi", A64, B64.sum(axis=1))
    tol = 8 * np.sqrt(C.shape[2]) * 2.0 ** -11 * float(np.abs(C64).max())
    assert np.abs(C64.sum(axis=2) - row_ref).max() <= tol
    if key == "bmm_f16_pv":
        # rows of P sum to one, so P.V of a constant V returns that constant (up to fp16 rounding of P)
        ones = np.ones_like(Bm)
        R = hostops.gemm(m, dev(A), dev(ones), group_m=gm).cpu().numpy()
        assert np.abs(R.astype(np.float32) - 1).max() < 5e-3


def test_conv2d_f16_full_size(hrn):
    m, gm = module("conv2d_f16")
    X, Wt = workloads.conv2d_inputs(32, 56, 56, 64, 64, 3, 3, seed=3)
    Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), 1, 1, 1, group_m=gm).cpu().numpy()
    for img in (0, 13, 31):
        ref = oracle.conv2d_nhwc_f32(X[img:img + 1], Wt, 1, 1, 1)
        check_f16(Y[img:img + 1], ref)
    # every output pixel: the sum over output channels equals the conv with the channel-summed filter
    Wsum = Wt.astype(np.float32).sum(axis=0, keepdims=True)
    ref = oracle.conv2d_nhwc_f32(X, Wsum, 1, 1, 1)[..., 0].astype(np.float64)
    Y64 = Y.astype(np.float64)
    assert np.abs(Y64.sum(axis=3) - ref).max() <= 8 * np.sqrt(64) * 2.0 ** -11 * float(np.abs(Y64).max())


def test_conv2d_u8s8_full_size(hrn):
    m, gm = module("conv2d_u8s8")
    X, Wt = workloads.conv2d_u8s8_inputs(32, 56, 56, 64, 64, 3, 3, seed=6)
    Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), 1, 1, 1, group_m=gm).cpu().numpy()
    for img in (0, 17, 31):
        assert np.array_equal(Y[img:img + 1], oracle.conv2d_nhwc_u8s8s32(X[img:img + 1], Wt, 1, 1, 1))
    # every output pixel, exactly: sum over output channels = conv with the channel-summed filter (fits float64 exactly)
    Wsum = Wt.astype(np.float32).sum(axis=0, keepdims=True)
    ref = oracle.conv2d_nhwc_f32(X.astype(np.float32), Wsum, 1, 1, 1)[..., 0].astype(np.int64)
    assert np.array_equal(Y.sum(axis=3, dtype=np.int64), ref)


def test_largest_operand_the_32_bit_offsets_allow(hrn):
    """One operand of a batch entry must stay below 2 GiB (buffer offsets are 32-bit): the largest A that fits is
    multiplied correctly (first, middle and last rows against the oracle), one row more is refused."""
    m = B.Module(instances.BEST["small_f16"])
    K, N = 16384, 64
    M = (2 ** 31 - 1) // (K * 2)                      # 65535 rows: 2 147 450 880 bytes
    rng = np.random.default_rng(5)
    Bm = (rng.normal(0, 0.1, (N, K))).astype(np.float16)
    A = torch.empty((M, K), dtype=torch.float16, device="cuda")
    A.normal_(0, 0.1)
    print("largest operand", (M, K, N), flush=True)
    C = hostops.gemm(m, A, dev(Bm))
    rows = [0, 1, M // 2, M - 2, M - 1]
    ref = oracle.gemm_f32(A[rows].cpu().numpy(), Bm)
    got = C[rows].cpu().numpy().astype(np.float32)
    check_f16(got, ref)
    del C
    A2 = torch.empty((M + 1, K), dtype=torch.float16, device="cuda")
    with pytest.raises(B.HeronRocmError):
        hostops.gemm(m, A2, dev(Bm))
