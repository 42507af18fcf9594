"""GPU parity of the operators declared as "pre-stage + product" (gemv, scan, mean, var, conv1d/2d/3d layouts,
dilated and transposed conv): operands in the reference's layouts go through the operand adapter and the MFMA
template, the result is compared with the float64 / int64 restatement of the reference declaration.

fp16: max|err| / max|ref| <= 1e-2 (fp16 inputs, fp32 accumulate, one rounding); integer forms bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from heron_amd import backend as B
from heron_amd import hostops, instances
from heron_amd.ops.rocm import getOpFromName
from parity_checks import check_f16

pytestmark = pytest.mark.gpu
REL_TOL = 1e-2
_mods = {}


class Ctx:
    def set_info(self, info):
        self.info = info

    def set_axis_map(self, m):
        self.axis_map = m


def declare(name, args, dtype):
    c = Ctx()
    out = getOpFromName(name)(c, *args, dtype, dtype)
    return c.info, out[0]


def module(info):
    f16 = info['kind'] == 'f16'
    if info['operator'] == 'conv2d_nhwc':
        d = instances.D(instances.F16, instances.CONV, *instances.PARITY_SHAPES[4]) if f16 else instances.int8_conv_descs()[0]
    else:
        d = instances.BEST["small_f16"] if f16 else instances.BEST["small"]
    key = d.as_tuple()
    if key not in _mods:
        _mods[key] = B.Module(d)
    return _mods[key]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rnd(shape, seed, dtype):
    rng = np.random.default_rng(seed)
    if dtype == "float16":
        return rng.normal(0, 1, shape).astype(np.float16)
    if dtype == "uint8":
        return rng.integers(0, 256, shape, dtype=np.uint8)
    return rng.integers(-128, 128, shape, dtype=np.int8)


def check(got, ref, f16):
    got = got.cpu().numpy()
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if f16:
        check_f16(got, ref)                 # tensor-level 1e-2 and the element-wise bound, as in the other suites
    else:
        assert got.dtype == np.int32 and np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_gemv_and_scan(dtype, hrn):
    f16 = dtype == "float16"
    a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
    for M, K in [(100, 72), (513, 1000), (64, 4096)]:
        info, out = declare("gemv", [M, K], dtype)
        A, b = rnd((M, K), 1, a_dt), rnd((1, K), 2, b_dt)
        print("gemv", dtype, M, K, flush=True)
        check(hostops.run_operator(module(info), info, [dev(A), dev(b)]), oracle.gemv_ref(A, b), f16)
    for M, N, K in [(64, 128, 128), (50, 40, 200), (7, 300, 104)]:
        info, out = declare("scan", [M, N, K], dtype)
        A = rnd((M, K), 3, a_dt)
        print("scan", dtype, M, N, K, flush=True)
        check(hostops.run_operator(module(info), info, [dev(A)]), oracle.scan_ref(A, N), f16)


def test_mean_and_var(hrn):
    for shape in [(4, 64, 14, 14), (3, 20, 7, 9), (1, 128, 28, 28)]:
        info, out = declare("mean", list(shape), "float16")
        In = rnd(shape, 4, "float16")
        print("mean/var", shape, flush=True)
        check(hostops.run_operator(module(info), info, [dev(In)]), oracle.mean_ref(In), True)
        Mean = np.broadcast_to(In.astype(np.float64).mean(axis=(0, 2, 3), keepdims=True), shape).astype(np.float16)
        info, out = declare("var", list(shape), "float16")
        check(hostops.run_operator(module(info), info, [dev(In), dev(Mean)]), oracle.var_ref(In, Mean), True)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_conv1d_layouts(dtype, hrn):
    f16 = dtype == "float16"
    a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
    for (N, W, CI, CO, K, s, p, d) in [(8, 100, 16, 32, 3, 1, 1, 1), (3, 57, 24, 20, 5, 2, 2, 1), (2, 64, 48, 8, 3, 1, 2, 2)]:
        X, F = rnd((N, W, CI), 5, a_dt), rnd((K, CI, CO), 6, b_dt)
        print("c1d", dtype, (N, W, CI, CO, K, s, p, d), flush=True)
        info, _ = declare("c1d_nwc", [N, W, CI, CO, K, s, p, d], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), oracle.conv1d_nwc_ref(X, F, s, p, d), f16)
        if d == 1:                                   # the NCW declaration asserts dilation == 1 (conv1d.py:17)
            info, _ = declare("c1d", [N, W, CI, CO, K, s, p, d], dtype)
            Xc, Fc = X.transpose(0, 2, 1), F.transpose(2, 1, 0)
            check(hostops.run_operator(module(info), info, [dev(Xc), dev(Fc)]), oracle.conv1d_ncw_ref(Xc, Fc, s, p, d), f16)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_conv2d_nchw_dilated_and_transposed(dtype, hrn):
    f16 = dtype == "float16"
    a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
    # first-layer shape with CI = 3 (channel padding), (h, w) pairs, plain
    for (N, H, W, CI, CO, KH, KW, s, p, d) in [(2, 20, 20, 3, 16, 7, 7, 2, 3, 1), (1, 12, 15, 16, 24, 3, 5, (2, 1), (1, 2), 1),
                                               (2, 9, 9, 32, 8, 3, 3, 1, 1, 1)]:
        X, F = rnd((N, CI, H, W), 7, a_dt), rnd((CO, CI, KH, KW), 8, b_dt)
        print("c2d_nchw", dtype, (N, H, W, CI, CO, KH, KW, s, p, d), flush=True)
        info, _ = declare("c2d_nchw", [N, H, W, CI, CO, KH, KW, s, p, d], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), oracle.conv2d_nchw_ref(X, F, s, p, d), f16)
    # channels-last conv whose channel count is short of a 16-byte chunk: padded by the adapter, result as it is
    for (N, H, W, CI, CO, KH, KW, s, p, d) in [(2, 20, 20, 3, 16, 7, 7, 2, 3, 1), (1, 9, 11, 20, 8, 3, 3, 1, 1, 1)]:
        X, F = rnd((N, H, W, CI), 15, a_dt), rnd((CO, KH, KW, CI), 16, b_dt)
        print("c2d short channels", dtype, (N, H, W, CI, CO, KH, KW, s, p, d), flush=True)
        info, _ = declare("c2d", [N, H, W, CI, CO, KH, KW, s, p, d], dtype)
        ref = oracle.conv2d_nhwc_f32(X, F, s, p, d) if f16 else oracle.conv2d_nhwc_u8s8s32(X, F, s, p, d)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), ref, f16)
        # the same call with the filter prepared once, as the measurer and a caller with fixed weights do
        weights = hostops.prepare_constant(info, [dev(X), dev(F)])
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)], constant=weights), ref, f16)
    for (N, H, W, CI, CO, KH, KW, s, p, d) in [(2, 20, 20, 16, 16, 3, 3, 1, 2, 2), (1, 17, 13, 8, 12, 3, 3, 2, 3, 3)]:
        X, F = rnd((N, H, W, CI), 9, a_dt), rnd((KH, KW, CI, CO), 10, b_dt)
        print("dil", dtype, (N, H, W, CI, CO, KH, KW, s, p, d), flush=True)
        info, _ = declare("dil", [N, H, W, CI, CO, KH, KW, s, p, d], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), oracle.dil_nhwc_ref(X, F, s, p, d), f16)
    for (N, H, W, CI, CO, KH, KW, s, p, d, op) in [(2, 7, 7, 16, 8, 4, 4, 2, 1, 1, 0), (1, 5, 6, 8, 12, 3, 3, 2, 1, 1, 1),
                                                   (2, 6, 5, 16, 4, 3, 3, 1, 0, 1, 0), (1, 4, 4, 16, 8, 3, 3, 3, 2, 2, 1)]:
        X, F = rnd((N, CI, H, W), 11, a_dt), rnd((CO, CI, KH, KW), 12, b_dt)
        print("t2d", dtype, (N, H, W, CI, CO, KH, KW, s, p, d, op), flush=True)
        info, _ = declare("t2d", [N, H, W, CI, CO, KH, KW, s, p, d, op], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]),
              oracle.conv2d_transposed_nchw_ref(X, F, s, p, d, op), f16)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_conv3d_layouts(dtype, hrn):
    f16 = dtype == "float16"
    a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
    for (N, D, H, W, CI, CO, KD, KH, KW, s, p, d) in [(2, 8, 10, 10, 16, 16, 3, 3, 3, 1, 1, 1),
                                                      (1, 6, 9, 7, 8, 12, 3, 3, 2, (2, 1, 1), (1, 1, 0), 1),
                                                      (1, 7, 8, 8, 16, 8, 2, 3, 3, 1, (0, 2, 1), (2, 2, 1))]:
        X, F = rnd((N, D, H, W, CI), 13, a_dt), rnd((KD, KH, KW, CI, CO), 14, b_dt)
        print("c3d", dtype, (N, D, H, W, CI, CO, KD, KH, KW, s, p, d), flush=True)
        info, _ = declare("c3d_ndhwc", [N, D, H, W, CI, CO, KD, KH, KW, s, p, d], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), oracle.conv3d_ndhwc_ref(X, F, s, p, d), f16)
        if d == 1:                                   # the NCDHW declaration asserts dilation == 1 (conv3d.py:15)
            Xc, Fc = X.transpose(0, 4, 1, 2, 3), F.transpose(4, 3, 0, 1, 2)
            info, _ = declare("c3d", [N, D, H, W, CI, CO, KD, KH, KW, s, p, d], dtype)
            check(hostops.run_operator(module(info), info, [dev(Xc), dev(Fc)]), oracle.conv3d_ncdhw_ref(Xc, Fc, s, p, d), f16)


def test_conv2d_nhwc_height_width_pairs(hrn):
    """(h, w) stride / padding / dilation pairs on the native NHWC operator, both element kinds."""
    for dtype in ("float16", "int8"):
        f16 = dtype == "float16"
        a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
        for (N, H, W, CI, CO, KH, KW, s, p, d) in [(1, 9, 12, 16, 16, 3, 2, (2, 1), (1, 0), (1, 2)), (2, 1, 33, 32, 8, 1, 3, (1, 2), (0, 2), 1),
                                                   (1, 10, 7, 16, 4, 2, 3, 1, (0, 1), (3, 1))]:
            X, Wt = rnd((N, H, W, CI), 15, a_dt), rnd((CO, KH, KW, CI), 16, b_dt)
            print("c2d pairs", dtype, (N, H, W, CI, CO, KH, KW, s, p, d), flush=True)
            info, _ = declare("c2d", [N, H, W, CI, CO, KH, KW, s, p, d], dtype)
            ref = oracle.conv2d_nhwc_f32(X, Wt, s, p, d).astype(np.float64) if f16 else oracle.conv2d_nhwc_u8s8s32(X, Wt, s, p, d)
            check(hostops.run_operator(module(info), info, [dev(X), dev(Wt)]), ref, f16)


@pytest.mark.parametrize("dtype", ["float16", "int8"])
def test_depthwise_conv(dtype, hrn):
    f16 = dtype == "float16"
    a_dt, b_dt = ("float16", "float16") if f16 else ("uint8", "int8")
    for (N, H, W, C, K, s, p) in [(2, 14, 14, 32, 32, 1, 1), (1, 17, 15, 24, 48, 2, 1), (2, 9, 9, 16, 48, 1, 0)]:
        X, F = rnd((N, C, H, W), 17, a_dt), rnd((K, 3, 3), 18, b_dt)
        print("dep", dtype, (N, H, W, C, K, s, p), flush=True)
        info, _ = declare("dep", [N, H, W, C, K, 3, 3, s, p, 1], dtype)
        check(hostops.run_operator(module(info), info, [dev(X), dev(F)]), oracle.depthwise_conv2d_ref(X, F, s, p), f16)


def test_pad_rows_kernel(hrn):
    """The channel-padding pre-stage of the library against torch's pad, both element sizes, odd row counts."""
    import torch
    for dtype, c, cp in [(torch.float16, 3, 8), (torch.float16, 20, 24), (torch.uint8, 3, 16), (torch.int8, 17, 32), (torch.float16, 1, 8)]:
        for rows in (1, 255, 4097):
            if dtype == torch.float16:
                t = torch.randn((rows, c), device="cuda").to(dtype)
            else:
                t = torch.randint(0, 100, (rows, c), device="cuda").to(dtype)
            out = torch.full((rows, cp), 7, dtype=dtype, device="cuda")
            B.pad_rows(t.data_ptr(), out.data_ptr(), rows, c, cp, t.element_size(), torch.cuda.current_stream().cuda_stream)
            torch.cuda.synchronize()
            assert torch.equal(out, torch.nn.functional.pad(t, (0, cp - c))), (dtype, c, cp, rows)
    x = torch.randn((2, 5, 7, 3), device="cuda").half()
    assert torch.equal(hostops._pad_last(x, 8), torch.nn.functional.pad(x, (0, 5)))
    with pytest.raises(B.HeronRocmError):
        B.pad_rows(x.data_ptr(), x.data_ptr(), 4, 3, 6, 2, 0)            # 12-byte rows are not whole 16-byte words


def test_transpose_pad_kernel(hrn):
    """The layout pre-/post-stage of the library against torch: three element sizes, sizes off the 64x64 tile, padding."""
    import torch
    st = torch.cuda.current_stream().cuda_stream
    for dtype in (torch.float16, torch.uint8, torch.int32):
        for (b, r, c, rp) in [(1, 3, 50, 8), (2, 64, 64, 64), (3, 65, 129, 72), (2, 20, 1000, 24), (1, 1, 1, 1), (4, 130, 7, 130)]:
            if dtype == torch.float16:
                x = torch.randn((b, r, c), device="cuda").to(dtype)
            else:
                x = torch.randint(0, 120, (b, r, c), device="cuda").to(dtype)
            out = torch.full((b, c, rp), 9, dtype=dtype, device="cuda")
            B.transpose_pad(x.data_ptr(), out.data_ptr(), b, r, c, rp, x.element_size(), st)
            torch.cuda.synchronize()
            ref = torch.nn.functional.pad(x.permute(0, 2, 1), (0, rp - r)).contiguous()
            assert torch.equal(out, ref), (dtype, b, r, c, rp)
    x = torch.randn((2, 5, 33), device="cuda").half()
    assert torch.equal(hostops._channels_last(x, 8), torch.nn.functional.pad(x.permute(0, 2, 1), (0, 3)))
    assert torch.equal(hostops._channels_first(x), x.permute(0, 2, 1).contiguous())
    with pytest.raises(B.HeronRocmError):
        B.transpose_pad(x.data_ptr(), x.data_ptr(), 1, 8, 8, 4, 2, st)             # padded rows fewer than rows
    with pytest.raises(B.HeronRocmError):
        B.transpose_pad(x.data_ptr(), x.data_ptr(), 1, 8, 8, 8, 3, st)             # 3-byte elements


def test_gather_kernel_against_the_torch_formulation(hrn):
    """The affine gather pass of the library (hrn_gather_nd): every adapter half that uses it, on device tensors, equals
    the torch formulation of the same pre-stage on the host copy bit for bit - 16-byte pieces (channel counts that are
    multiples of 8, aligned maps) and single elements (everything else), fp16 and bytes, the fused (x - mean)^2 included."""
    import torch

    def both(fn, name, args, dtype, *host):
        info, _ = declare(name, args, dtype)
        print("gather", name, args, dtype, flush=True)
        want = fn(info, *[torch.from_numpy(np.ascontiguousarray(h)) for h in host])
        got = fn(info, *[dev(h) for h in host])
        torch.cuda.synchronize()
        assert got.is_cuda and got.is_contiguous() and got.shape == want.shape
        assert torch.equal(got.cpu(), want), (name, args)

    for shape in [(4, 64, 14, 14), (3, 20, 7, 9), (1, 5, 3, 3), (2, 16, 8, 8)]:
        In, Mean = rnd(shape, 30, "float16"), rnd(shape, 31, "float16")
        both(hostops._act_mean, "mean", list(shape), "float16", In)
        both(hostops._act_var, "var", list(shape), "float16", In, Mean)
    for dtype in ("float16", "int8"):
        adt = "float16" if dtype == "float16" else "uint8"
        for ci in (5, 8, 16):
            for s, p, d in [(1, 1, 1), ((2, 1, 1), (1, 1, 0), 1), (1, (0, 2, 1), (2, 2, 1))]:
                X, F = rnd((2, 6, 9, 7, ci), 32, adt), rnd((3, 3, 2, ci, 16), 33, dtype)
                both(hostops._act_c3d_ndhwc, "c3d_ndhwc", [2, 6, 9, 7, ci, 16, 3, 3, 2, s, p, d], dtype, X, F)
        for ci in (6, 16):
            for s, p, d, op in [(2, 1, 1, 0), (2, 1, 1, 1), (1, 0, 1, 0), (3, 2, 2, 1)]:
                X, F = rnd((2, ci, 5, 6), 34, adt), rnd((4, ci, 3, 4), 35, dtype)
                both(hostops._act_t2d_nchw, "t2d", [2, 5, 6, ci, 4, 3, 4, s, p, d, op], dtype, X, F)
        for s, p, mult in [(1, 1, 1), (2, 1, 2)]:
            X, F = rnd((2, 6, 9, 8), 36, adt), rnd((6 * mult, 3, 3), 37, dtype)
            both(hostops._act_dep, "dep", [2, 9, 8, 6, 6 * mult, 3, 3, s, p, 1], dtype, X, F)
    # argument checks
    x = torch.zeros(64, dtype=torch.float16, device="cuda")
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})])
    B.gather_nd(g, x.data_ptr(), x.data_ptr())
    g.dst_stride[1] = 2
    with pytest.raises(B.HeronRocmError, match="stride 1"):
        B.gather_nd(g, x.data_ptr(), x.data_ptr())
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})], op=B.GATHER_CENTER_SQUARE)
    with pytest.raises(B.HeronRocmError, match="aux"):
        B.gather_nd(g, x.data_ptr(), x.data_ptr())
    g = B.make_gather(3, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})])
    with pytest.raises(B.HeronRocmError):
        B.gather_nd(g, x.data_ptr(), x.data_ptr())


def test_operator_plans_replay_what_run_operator_does(hrn):
    """hostops.OperatorPlan: recorded once, every replay leaves in the plan's result tensor exactly what an eager
    run_operator computes from the inputs' current contents - also after the inputs were overwritten in place (the
    plan's own validation does that once; here it is done again with fresh data) - for every kind of adapter."""
    import torch
    cases = [
        ("gemv", [100, 72], "float16", [(100, 72), (1, 72)]),
        ("scan", [33, 40, 100], "float16", [(33, 100)]),
        ("mean", [3, 20, 7, 9], "float16", [(3, 20, 7, 9)]),
        ("var", [3, 20, 7, 9], "float16", [(3, 20, 7, 9), (3, 20, 7, 9)]),
        ("c1d", [3, 57, 12, 20, 5, 2, 2, 1], "float16", [(3, 12, 57), (20, 12, 5)]),
        ("c2d_nchw", [2, 20, 20, 3, 16, 7, 7, 2, 3, 1], "float16", [(2, 3, 20, 20), (16, 3, 7, 7)]),
        ("c2d", [2, 20, 20, 3, 16, 7, 7, 2, 3, 1], "float16", [(2, 20, 20, 3), (16, 7, 7, 3)]),
        ("c3d_ndhwc", [2, 6, 9, 7, 5, 12, 3, 3, 2, 1, 1, 1], "float16", [(2, 6, 9, 7, 5), (3, 3, 2, 5, 12)]),
        ("c3d", [2, 6, 9, 7, 8, 16, 3, 3, 2, 1, 1, 1], "int8", [(2, 8, 6, 9, 7), (16, 8, 3, 3, 2)]),
        ("t2d", [2, 5, 6, 6, 4, 3, 4, 2, 1, 1, 1], "float16", [(2, 6, 5, 6), (4, 6, 3, 4)]),
        ("dep", [2, 9, 8, 6, 12, 3, 3, 2, 1, 1], "float16", [(2, 6, 9, 8), (12, 3, 3)]),
        ("gemm", [70, 144, 48], "int8", [(70, 144), (48, 144)]),
    ]
    for name, args, dtype, shapes in cases:
        info, _ = declare(name, args, dtype)
        adt = "float16" if dtype == "float16" else "uint8"
        inputs = [dev(rnd(sh, 40 + i, adt if i == 0 else dtype)) for i, sh in enumerate(shapes)]
        mod = module(info)
        print("plan", name, args, dtype, flush=True)
        plan = hostops.OperatorPlan(mod, info, inputs)
        assert plan.steps and torch.equal(plan.run(), hostops.run_operator(mod, info, inputs, constant=plan.constant))
        inputs[0].copy_(dev(rnd(shapes[0], 77, adt)))
        want = hostops.run_operator(mod, info, inputs, constant=plan.constant)
        got = plan.run()
        torch.cuda.synchronize()
        assert got is plan.out and torch.equal(got, want), name
