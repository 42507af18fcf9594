"""Benchmark of the MFMA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One step = one launch of the tuned template instance over a batch of synthetic operands that are
already resident in HBM.  Prints ONE JSON line.  The headline workload is the dense fp16 GEMM
M=N=K=4096 (fp32 accumulate, fp16 output); the other benchmark configurations are reported under
"also" in the same line.  `roofline.achieved` is algorithmic work per launch divided by the average
kernel duration measured with HIP events on the launch stream.  `cpu_baseline` times the CPU oracle
(the DL Boost-style VNNI GEMM for the quantized case, the fp32 host reference otherwise) on a bounded
sample of the same workload, on this machine's host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def make_workloads(torch, workloads, instances):
    """name -> dict(desc, problem factory, device operands, ops, bytes, peak, dtype)."""
    from heron_amd import backend as B

    def dev(a):
        return torch.from_numpy(a).cuda()

    W = {}

    def add_gemm(name, key, M, K, N, f16, batch=1, gen=None):
        group_m = instances.BEST_GROUP_M.get(key, 8)

        def build():
            if gen is not None:
                A, Bm = gen()
            elif f16:
                A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=1)
            else:
                A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=2)
            shape = (batch, M, N) if batch > 1 else (M, N)
            C = torch.empty(shape, dtype=torch.float16 if f16 else torch.int32, device="cuda")
            return dev(A), dev(Bm), C, B.gemm_problem(batch, M, N, K, group_m)
        ops, byts = workloads.gemm_work(M, N, K, 2 if f16 else 1, 2 if f16 else 4, batch)
        W[name] = dict(desc=instances.BEST[key], build=build, ops=ops, bytes=byts, f16=f16,
                       desc_text="%s batch=%d M=%d N=%d K=%d" % ("gemm_f16" if f16 else "gemm_u8s8", batch, M, N, K))

    add_gemm("gemm_f16_4096", "gemm_f16_4096", 4096, 4096, 4096, True)
    add_gemm("gemm_f16_8192", "gemm_f16", 8192, 8192, 8192, True)
    add_gemm("gemm_u8s8_8192", "gemm_u8s8", 8192, 8192, 8192, False)
    add_gemm("bmm_f16_qk", "bmm_f16_qk", 512, 64, 512, True, 192, lambda: workloads.bmm_qk_inputs(192, 512, 64, 512))
    add_gemm("bmm_f16_pv", "bmm_f16_pv", 512, 512, 64, True, 192, lambda: workloads.bmm_pv_inputs(192, 512, 512, 64))

    def build_conv():
        X, Wt = workloads.conv2d_inputs(32, 56, 56, 64, 64, 3, 3, seed=3)
        Y = torch.empty((32, 56, 56, 64), dtype=torch.float16, device="cuda")
        return dev(X), dev(Wt), Y, B.conv2d_problem(32, 56, 56, 64, 64, 3, 3, 1, 1, 1,
                                                    instances.BEST_GROUP_M.get("conv2d_f16", 8))
    ops, byts = workloads.conv_work(32, 56, 56, 64, 64, 3, 3, 1, 1, 1)
    W["conv2d_f16_resnet"] = dict(desc=instances.BEST["conv2d_f16"], build=build_conv, ops=ops, bytes=byts, f16=True,
                                  desc_text="conv2d_nhwc_f16 N=32 H=W=56 C=64 K=64 3x3 s1 p1")

    def build_conv_i8():
        X, Wt = workloads.conv2d_u8s8_inputs(32, 56, 56, 64, 64, 3, 3, seed=6)
        Y = torch.empty((32, 56, 56, 64), dtype=torch.int32, device="cuda")
        return dev(X), dev(Wt), Y, B.conv2d_problem(32, 56, 56, 64, 64, 3, 3, 1, 1, 1,
                                                    instances.BEST_GROUP_M.get("conv2d_u8s8", 8))
    ops, byts = workloads.conv_work(32, 56, 56, 64, 64, 3, 3, 1, 1, 1, in_bytes=1, out_bytes=4)
    W["conv2d_u8s8_resnet"] = dict(desc=instances.BEST["conv2d_u8s8"], build=build_conv_i8, ops=ops, bytes=byts, f16=False,
                                   desc_text="conv2d_nhwc_u8s8 N=32 H=W=56 C=64 K=64 3x3 s1 p1")
    return W


def measure(torch, B, w, steps, warmup, keep_rows=0):
    """Returns (wall seconds per step, event seconds per launch, kernel resources[, first rows of the timed output])."""
    mod = B.Module(w["desc"])
    a, b, c, prob = w["build"]()
    stream = torch.cuda.current_stream().cuda_stream
    if warmup > 0:
        mod.launch_repeat(prob, a.data_ptr(), b.data_ptr(), c.data_ptr(), warmup, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    mod.launch_repeat(prob, a.data_ptr(), b.data_ptr(), c.data_ptr(), steps, stream)     # exactly `steps` launches
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    # per-launch kernel duration from HIP events recorded on the launch stream
    costs = mod.time(prob, a.data_ptr(), b.data_ptr(), c.data_ptr(), number=steps, repeat=3, min_repeat_ms=0.0, stream=stream)
    ev = sorted(costs)[len(costs) // 2]
    info = dict(mod.info)
    mod.close()
    rows = c.reshape(-1, c.shape[-1])[:keep_rows].cpu().numpy() if keep_rows else None
    del a, b, c
    return (wall, ev, info, rows) if keep_rows else (wall, ev, info)


# HBM bytes per launch of the dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by
# what the same counters read for the plain copy kernel of known size (profiles/ holds the runs these come from)
MEASURED_TRAFFIC = {
    "gemm_f16_4096": 235.0e6,     # profiles/hrn_mfma_kernel_gemm_f16_4096.md
    "gemm_f16_8192": 1746.1e6,    # profiles/hrn_mfma_kernel_gemm_f16_8192.md
    "gemm_u8s8_8192": 1074.4e6,   # profiles/hrn_mfma_kernel_gemm_u8s8_8192.md
    "bmm_f16_qk": 126.0e6,        # profiles/hrn_mfma_kernel_conv_bmm.md
    "conv2d_f16_resnet": 26.5e6,  # profiles/hrn_mfma_kernel_conv_bmm.md
    "bmm_f16_pv": 125.9e6,        # profiles/hrn_mfma_kernel_conv_bmm.md
    "conv2d_u8s8_resnet": 32.6e6, # profiles/hrn_mfma_kernel_conv_bmm.md
}


def safe_probes(torch, B):
    try:
        return run_probes(torch, B)
    except Exception as e:  # noqa: BLE001 - context figures only
        return {"error": repr(e)[:200]}


def run_probes(torch, B):
    """Roofline denominators measured on this GPU next to the published ones."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda")
    dst = torch.empty(n, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    out = {
        "mfma_f16_const_operands_TFLOPs": B.probe_mfma(B.HRN_DT_F16, 32, False, st),
        "mfma_f16_random_operands_TFLOPs": B.probe_mfma(B.HRN_DT_F16, 32, True, st),
        "mfma_i8_const_operands_TOPs": B.probe_mfma(B.HRN_DT_U8S8, 32, False, st),
        "mfma_i8_random_operands_TOPs": B.probe_mfma(B.HRN_DT_U8S8, 32, True, st),
        "hbm_copy_1GiB_read_plus_write_GBs": B.probe_copy(src.data_ptr(), dst.data_ptr(), n, 10, st),
    }
    del src, dst
    # the vendor library on the same random operands, for orientation only (torch.matmul = hipBLASLt / rocBLAS);
    # a library problem must not cost the benchmark line
    try:
        for n in (4096, 8192):
            a = (torch.randn(n, n, device="cuda") * 0.1).half()
            b = (torch.randn(n, n, device="cuda") * 0.1).half()
            for _ in range(5):
                torch.matmul(a, b.t())
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 200 if n == 4096 else 50
            e0.record()
            for _ in range(reps):
                torch.matmul(a, b.t())
            e1.record()
            torch.cuda.synchronize()
            out["vendor_library_gemm_f16_%d_TFLOPs" % n] = 2.0 * n ** 3 / (e0.elapsed_time(e1) * 1e-3 / reps) / 1e12
            del a, b
    except Exception as e:  # noqa: BLE001
        out["vendor_library_error"] = repr(e)[:200]
    # the library's int8 product (signed x signed -> int32, the closest it offers to the u8 x s8 GEMM) on random bytes
    try:
        n = 8192
        a = torch.randint(-128, 128, (n, n), device="cuda", dtype=torch.int8)
        b = torch.randint(-128, 128, (n, n), device="cuda", dtype=torch.int8)
        for _ in range(5):
            torch._int_mm(a, b.t())
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            torch._int_mm(a, b.t())
        e1.record()
        torch.cuda.synchronize()
        out["vendor_library_gemm_s8s8_8192_TOPs"] = 2.0 * n ** 3 / (e0.elapsed_time(e1) * 1e-3 / 50) / 1e12
        del a, b
    except Exception as e:  # noqa: BLE001
        out["vendor_library_int8_error"] = repr(e)[:200]
    # the library's convolution (torch conv2d = MIOpen) on the ResNet-50 stage-2 shape, channels-last fp16 in and out
    try:
        x = torch.relu(torch.randn(32, 64, 56, 56, device="cuda")).half().contiguous(memory_format=torch.channels_last)
        w = (torch.randn(64, 64, 3, 3, device="cuda") * 0.05).half().contiguous(memory_format=torch.channels_last)
        for _ in range(20):            # the library's first calls of a shape run a slow fallback kernel
            torch.nn.functional.conv2d(x, w, padding=1)
        torch.cuda.synchronize()
        groups = []
        for _ in range(5):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(100):
                torch.nn.functional.conv2d(x, w, padding=1)
            e1.record()
            torch.cuda.synchronize()
            groups.append(e0.elapsed_time(e1) * 1e3 / 100)
        out["vendor_library_conv2d_f16_resnet_us"] = min(groups)
        del x, w
    except Exception as e:  # noqa: BLE001
        out["vendor_library_conv_error"] = repr(e)[:200]
    return out


def roofline(w, ev_seconds, workloads):
    ai = w["ops"] / w["bytes"]
    peak_mfma = workloads.PEAK_FP16_TFLOPS if w["f16"] else workloads.PEAK_INT8_TOPS
    ridge = peak_mfma * 1e12 / (workloads.PEAK_HBM_GBS * 1e9)
    if ai >= ridge:
        ach = w["ops"] / ev_seconds / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": peak_mfma, "unit": "TFLOP/s" if w["f16"] else "TOP/s",
                "frac": ach / peak_mfma, "traffic": None}
    ach = w["bytes"] / ev_seconds / 1e9
    return {"bound": "hbm", "achieved": ach, "peak": workloads.PEAK_HBM_GBS, "unit": "GB/s",
            "frac": ach / workloads.PEAK_HBM_GBS, "traffic": None}


def cpu_baseline(name, workloads, gpu_rows=None):
    """The CPU oracle on a bounded sample of the workload (checker code used as a reported baseline only).  When the
    first rows of the GPU output of the timed buffers are passed in, the same sample also checks them."""
    import numpy as np
    import oracle
    cores = len(os.sched_getaffinity(0))
    if name.startswith("gemm_u8s8"):
        M, K, N = 8192, 8192, 8192
        A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=2)
        if oracle.has_vnni():
            pb = oracle.PackedB(Bm)
            C = np.empty((M, N), np.int32)
            pb.matmul(A[:256], out=C[:256])                # warm-up
            reps, t0 = 0, time.perf_counter()
            while True:
                pb.matmul(A, out=C)
                reps += 1
                if time.perf_counter() - t0 > 10 or reps >= 20:
                    break
            dt = (time.perf_counter() - t0) / reps
            out = {"value": 2.0 * M * N * K / dt / 1e12, "unit": "TOP/s", "cores": oracle.num_threads(), "kind": "port",
                   "sample": "full 8192^3 u8s8 GEMM x%d, AVX512-VNNI 16x4 vpdpbusd micro-kernel, B pre-packed, "
                             "%d OpenMP threads of %d host cores" % (reps, oracle.num_threads(), cores)}
            if gpu_rows is not None:
                out["gpu_rows_bit_exact"] = bool(np.array_equal(gpu_rows, C[:len(gpu_rows)]))
            return out
        rows = 64
        t0 = time.perf_counter()
        oracle.gemm_u8s8s32_dlboost(A[:rows], Bm)
        dt = time.perf_counter() - t0
        return {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TOP/s", "cores": oracle.num_threads(), "kind": "port",
                "sample": "%d rows of the 8192^3 u8s8 GEMM, scalar fallback (no AVX512-VNNI)" % rows}
    # fp16 workloads: fp32 host reference (double accumulate) on a slab of rows
    M, K, N = 4096, 4096, 4096
    A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=1)
    rows = 64
    Af, Bf = A[:rows].astype(np.float32), Bm.astype(np.float32)
    oracle.gemm_f32(Af[:8], Bf)
    t0 = time.perf_counter()
    reps = 0
    while True:
        oracle.gemm_f32(Af, Bf)
        reps += 1
        if time.perf_counter() - t0 > 10 or reps >= 50:
            break
    dt = (time.perf_counter() - t0) / reps
    out = {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
           "sample": "%d of 4096 rows of the fp16 GEMM 4096^3 x%d, fp32 host reference (double accumulate), "
                     "%d OpenMP threads of %d host cores" % (rows, reps, oracle.num_threads(), cores)}
    if gpu_rows is not None:
        ref = oracle.gemm_f32(Af[:len(gpu_rows)], Bf)
        out["gpu_rows_max_rel_err"] = float(np.abs(gpu_rows.astype(np.float32) - ref).max() / np.abs(ref).max())
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="gemm_f16_4096")
    ap.add_argument("--only", action="store_true", help="skip the 'also' workloads and the CPU baseline")
    ap.add_argument("--probe", action="store_true", help="only run the roofline probes (MFMA loop, 1 GiB copy)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path is a single-GPU kernel and no multi-GPU figure is produced "
              "(got --gpus %d)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from heron_amd import backend as B
    from heron_amd import instances, workloads
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    B.lib()
    if args.probe:
        print(json.dumps({"probes": run_probes(torch, B)}))
        return
    W = make_workloads(torch, workloads, instances)
    if args.workload not in W:
        print("unknown workload %s (have %s)" % (args.workload, sorted(W)), file=sys.stderr)
        sys.exit(2)

    w = W[args.workload]
    check_rows = 64 if (args.workload in ("gemm_f16_4096", "gemm_u8s8_8192") and not args.only) else 0
    if check_rows:
        wall, ev, info, gpu_rows = measure(torch, B, w, args.steps, args.warmup, check_rows)
    else:
        (wall, ev, info), gpu_rows = measure(torch, B, w, args.steps, args.warmup), None
    line = {
        "metric": "%s throughput per GPU (tuned MFMA template)" % ("fp16 GEMM TFLOPS" if w["f16"] else "u8s8 GEMM TOPS"),
        "value": w["ops"] / wall / 1e12,
        "unit": "TFLOP/s" if w["f16"] else "TOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if w["f16"] else "u8",
        "data": "synthetic",
        "config": {"workload": w["desc_text"], "instance": repr(w["desc"]), "kernel_ms": ev * 1e3, "resources": info},
        "roofline": roofline(w, ev, workloads),
    }
    line["roofline"]["traffic"] = MEASURED_TRAFFIC.get(args.workload)
    line["peaks"] = {"published": {"mfma_f16_TFLOPs": workloads.PEAK_FP16_TFLOPS, "mfma_i8_TOPs": workloads.PEAK_INT8_TOPS,
                                   "hbm_GBs": workloads.PEAK_HBM_GBS},
                     "measured": safe_probes(torch, B), "used": "published"}
    if not args.only:
        also = []
        for name, ww in W.items():
            if name == args.workload:
                continue
            steps = max(10, min(args.steps, 500))
            try:
                wl, e, _ = measure(torch, B, ww, steps, min(args.warmup, 5))
            except Exception as err:  # noqa: BLE001 - one side workload must not cost the headline
                also.append({"workload": ww["desc_text"], "error": repr(err)[:200]})
                continue
            r = roofline(ww, e, workloads)
            r["traffic"] = MEASURED_TRAFFIC.get(name)
            also.append({"workload": ww["desc_text"], "value": ww["ops"] / wl / 1e12,
                         "unit": "TFLOP/s" if ww["f16"] else "TOP/s", "steps": steps, "kernel_ms": e * 1e3,
                         "frac_of_mfma_peak": ww["ops"] / e / 1e12 / (workloads.PEAK_FP16_TFLOPS if ww["f16"] else workloads.PEAK_INT8_TOPS),
                         "roofline": r})
        line["also"] = also
        def guarded(*a):
            try:
                return cpu_baseline(*a)
            except Exception as e:  # noqa: BLE001 - the GPU figures above are still worth printing
                return {"value": None, "unit": None, "cores": 0, "kind": "port", "sample": "failed: %r" % (e,)}
        line["cpu_baseline"] = guarded(args.workload, workloads, gpu_rows)
        line["cpu_baseline_u8s8"] = guarded("gemm_u8s8_8192", workloads) if not args.workload.startswith("gemm_u8s8") else None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
