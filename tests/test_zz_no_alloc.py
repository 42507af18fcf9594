"""The allocation-free split-K entry point (hrn_launch_splitk_static) against the entry points that take a caller-owned
workspace: same kernels, same slices, so the outputs must be identical bit for bit (and the uint8 path equal to the
oracle).  Two calls in a row share the library's one static workspace per GPU; the second has the smaller input, so
stale partial sums of the first lie behind its own.  Sizes beyond the static workspace are refused."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from heron_amd import backend as B
from heron_amd import instances, workloads
from parity_checks import check_f16

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(a).cuda()


def both_ways(mod, f16, M, K, N, split, seed):
    A, Bm = (workloads.gemm_f16_inputs if f16 else workloads.gemm_u8s8_inputs)(M, K, N, seed=seed)
    a, b = dev(A), dev(Bm)
    odt = torch.float16 if f16 else torch.int32
    c_ws = torch.full((M, N), -7, dtype=odt, device="cuda")
    c_st = torch.full((M, N), -9, dtype=odt, device="cuda")
    p = B.gemm_problem(1, M, N, K, 8, split_k=split)
    mod.launch(p, a.data_ptr(), b.data_ptr(), c_ws.data_ptr())                  # caller-owned workspace (module's buffer)
    q = B.gemm_problem(1, M, N, K, 8, split_k=split)                            # no workspace bound at all
    assert not q.workspace
    print("no-alloc split-K", mod.desc.as_tuple(), (M, K, N), split, flush=True)
    mod.launch_splitk_static(q, a.data_ptr(), b.data_ptr(), c_st.data_ptr())
    torch.cuda.synchronize()
    return A, Bm, c_ws.cpu().numpy(), c_st.cpu().numpy()


@pytest.mark.parametrize("f16", [True, False], ids=["f16", "u8s8"])
def test_static_workspace_matches_caller_workspace(f16, hrn):
    desc = [d for d in instances.splitk_descs() if d.op == instances.GEMM and (d.dtype == instances.F16) == f16][0]
    mod = B.Module(desc)
    # first call: larger problem; second call right behind it: smaller, fewer slices
    for (M, K, N, split, seed) in [(784, 4608, 512, 8, 1), (100, 1040, 72, 3, 2)]:
        A, Bm, got_ws, got_st = both_ways(mod, f16, M, K, N, split, seed)
        assert np.array_equal(got_ws, got_st)
        if f16:
            check_f16(got_st, oracle.gemm_f32(A, Bm))
        else:
            assert np.array_equal(got_st, oracle.gemm_int64_numpy(A, Bm).astype(np.int32))
    mod.close()


def test_static_workspace_allocates_nothing_and_serialises_streams(hrn):
    """The entry point takes no device memory (the driver's free-memory figure and torch's allocator are unchanged
    across calls), also for a batched uint8 problem; and two calls issued back to back on two different streams -
    which share the one workspace - are ordered by the library: both results equal the caller-workspace results."""
    desc = [d for d in instances.splitk_descs() if d.op == instances.GEMM and d.dtype == instances.U8 and not d.colsum][0]
    mod = B.Module(desc)
    rng = np.random.default_rng(3)
    cases = []
    for (b, M, K, N, split) in [(3, 200, 2064, 136, 4), (1, 784, 4608, 256, 8)]:
        A = rng.integers(0, 256, (b, M, K), dtype=np.uint8)
        Bm = rng.integers(-128, 128, (b, N, K), dtype=np.int8)
        a, bb = dev(A), dev(Bm)
        ref = torch.empty((b, M, N), dtype=torch.int32, device="cuda")
        p = B.gemm_problem(b, M, N, K, 8, split_k=split)
        mod.launch(p, a.data_ptr(), bb.data_ptr(), ref.data_ptr())
        out = torch.full((b, M, N), -5, dtype=torch.int32, device="cuda")
        cases.append((a, bb, out, ref, B.gemm_problem(b, M, N, K, 8, split_k=split), A, Bm))
    torch.cuda.synchronize()
    assert np.array_equal(cases[0][3].cpu().numpy(), oracle.bmm_u8s8s32_scalar(cases[0][5], cases[0][6]))
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for (a, bb, out, ref, q, _, _), st in zip(cases, (s1, s2)):          # the streams' own queues come into being here
        mod.launch_splitk_static(q, a.data_ptr(), bb.data_ptr(), out.data_ptr(), st.cuda_stream)
    torch.cuda.synchronize()
    for c in cases:
        c[2].fill_(-5)
    torch.cuda.synchronize()
    free0, alloc0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for rounds in range(3):
        for (a, bb, out, ref, q, _, _), st in zip(cases, (s1, s2)):
            mod.launch_splitk_static(q, a.data_ptr(), bb.data_ptr(), out.data_ptr(), st.cuda_stream)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == alloc0
    assert torch.cuda.memory_reserved() == reserved0
    for (a, bb, out, ref, q, _, _) in cases:
        assert torch.equal(out, ref)
    mod.close()


def test_static_workspace_limits(hrn):
    desc = instances.splitk_descs()[0]
    mod = B.Module(desc)
    L = B.lib()
    M, K, N = 2048, 1024, 2048                    # 4 slices x 2048 x 2048 x 4 bytes = 64 MiB > 32 MiB
    a = torch.zeros((M, K), dtype=torch.float16, device="cuda")
    b = torch.zeros((N, K), dtype=torch.float16, device="cuda")
    c = torch.zeros((M, N), dtype=torch.float16, device="cuda")
    p = B.gemm_problem(1, M, N, K, 8, split_k=4)
    assert B.splitk_workspace_bytes(desc, p) > B.STATIC_WORKSPACE_BYTES
    assert L.hrn_launch_splitk_static(mod._h, ctypes.byref(p), a.data_ptr(), b.data_ptr(), c.data_ptr(), 0) == B.HRN_E_BADPARAM
    assert b"static workspace" in L.hrn_last_error()
    # an instance without split_k has no partial sums to park
    plain = B.Module(instances.BEST["small_f16"])
    p1 = B.gemm_problem(1, 64, 64, 64, 8)
    assert L.hrn_launch_splitk_static(plain._h, ctypes.byref(p1), a.data_ptr(), b.data_ptr(), c.data_ptr(), 0) == B.HRN_E_BADPARAM
    plain.close()
    mod.close()
