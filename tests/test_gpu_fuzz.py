"""GPU parity of template instances drawn from the tuner's own search space (tests/golden/fuzz_instances.json, made by
tests/golden/make_fuzz_instances.py with a fixed seed): knob combinations nobody picked by hand - odd per-wave tile
counts, five stages, one k-step per tile, persistent launches, window mode, split-K - against the oracle on ragged shapes.
Integer results bit-exact, fp16 within rel. error 1e-2.
"""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from heron_amd import backend as B
from heron_amd import hostops, instances, workloads
from parity_checks import check_f16

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
FUZZ = json.load(open(os.path.join(HERE, "golden", "fuzz_instances.json")))

GEMM_SHAPES = [(300, 1024, 520), (2048, 320, 512), (64, 4096, 136)]                       # (M, K, N)
CONV_CASES = [(2, 14, 14, 64, 64, 3, 3, 1, 1, 1), (1, 30, 30, 32, 64, 3, 3, 2, 1, 1), (3, 9, 11, 128, 48, 3, 3, 1, 1, 1),
              (2, 16, 16, 256, 32, 1, 1, 1, 0, 1)]


def dev(a):
    return torch.from_numpy(a).cuda()


def close(got, ref, f16):
    if f16:
        check_f16(got, ref)
    else:
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("entry", FUZZ, ids=lambda e: "-".join(map(str, e["desc"])))
def test_sampled_instance(entry, hrn):
    d = B.make_desc(*entry["desc"])
    gm, sk = entry["group_m"], entry["split_k"]
    m = B.Module(d)
    assert m.info["scratch_bytes"] >= 0
    f16 = d.dtype == instances.F16
    ran = 0
    if d.op == instances.GEMM:
        for i, (M, K, N) in enumerate(GEMM_SHAPES):
            print("fuzz gemm", entry["desc"], (M, K, N), flush=True)
            if f16:
                A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=200 + i)
                close(hostops.gemm(m, dev(A), dev(Bm), group_m=gm, split_k=sk).cpu().numpy(), oracle.gemm_f32(A, Bm), True)
            else:
                A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=200 + i)
                close(hostops.gemm(m, dev(A), dev(Bm), group_m=gm, split_k=sk).cpu().numpy(), oracle.gemm_int64_numpy(A, Bm), False)
            ran += 1
    else:
        for i, case in enumerate(CONV_CASES):
            N, H, W, CI, CO, KH, KW, s, p, dl = case
            es = 2 if f16 else 1
            print("fuzz conv", entry["desc"], case, flush=True)
            gen = workloads.conv2d_inputs if f16 else workloads.conv2d_u8s8_inputs
            X, Wt = gen(N, H, W, CI, CO, KH, KW, seed=210 + i)
            window_ok = s == 1 and dl == 1 and 2 * p == KH - 1 and (CI * es) % d.bkb == 0
            if d.conv_window and not window_ok:
                with pytest.raises(B.HeronRocmError):
                    hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, dl, group_m=gm, split_k=sk)
                continue
            try:
                Y = hostops.conv2d_nhwc(m, dev(X), dev(Wt), s, p, dl, group_m=gm, split_k=sk).cpu().numpy()
            except B.HeronRocmError as e:
                assert d.conv_window and "exceeds 163840" in str(e)          # window + static LDS too large for this image width
                continue
            ref = oracle.conv2d_nhwc_f32(X, Wt, s, p, dl) if f16 else oracle.conv2d_nhwc_u8s8s32(X, Wt, s, p, dl)
            close(Y, ref, f16)
            ran += 1
    assert ran >= 1
    m.close()
