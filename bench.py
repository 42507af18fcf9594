"""Benchmark of the MFMA hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

One step = one launch of the tuned template instance over a batch of synthetic operands that are already resident in
HBM.  Prints ONE JSON line.  The headline workload is the quantized GEMM M=N=K=8192 (uint8 x int8 -> int32); the other
benchmark configurations are reported under "also" in the same line.  Every instance is the best record of
tests/quick_start/rocm/tuned/<case>/records.txt, replayed through Task.apply_best.

Timing.  Before anything is timed the same kernel runs untimed until the chip's clocks have settled (at least 200 ms,
then until two consecutive 20-launch groups agree within 2 %); this does not depend on --warmup.  Then --warmup untimed
launches, then exactly --steps launches bracketed by torch.cuda.synchronize() for ``value`` / ``ms_per_step`` and by
HIP events on the launch stream for ``config.kernel_ms`` (what ``roofline.achieved`` is computed from).  Rows bounded by
HBM are also timed cold - every launch after 1 GiB was streamed through the caches - and their roofline fraction
is the cold one: back-to-back launches of a 126 MB problem run out of the 256 MB memory-side cache.  Next to it stands
the like-for-like floor of such a launch: a kernel that only reads the workload's input bytes and writes its output
bytes, one launch after the same flush (``floor_us_cold``, ``frac_of_floor``).

A uint8 instance may take the column sums of B with the weights (``colsum`` instances): they depend on the weights
alone, as the reference's pre-packed weight operand does, and are made once, outside the timed region; the line says
so (``config.weights``) and also gives the figure with that pass counted into every step (``with_colsum_pass``).
``stable`` repeats the three GEMM figures under fixed names, whichever workload is the headline.

``cpu_baseline`` times the CPU oracle's DL Boost-style GEMM (AVX512-VNNI 16x4 micro-kernel, all host cores) on the
same 8192^3 problem and checks the first rows of the very buffer that was timed against it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HEADLINE = "gemm_u8s8_8192"


def make_workloads(torch, workloads, tuned):
    """name -> dict(instance, problem factory, ops, bytes, f16, text)."""
    from heron_amd import backend as B

    def dev(a):
        return torch.from_numpy(a).cuda()

    W = {}

    def add_gemm(name, M, K, N, f16, batch=1, gen=None):
        inst = tuned.load(name)

        def build():
            if gen is not None:
                A, Bm = gen()
            elif f16:
                A, Bm = workloads.gemm_f16_inputs(M, K, N, seed=1)
            else:
                A, Bm = workloads.gemm_u8s8_inputs(M, K, N, seed=2)
            shape = (batch, M, N) if batch > 1 else (M, N)
            C = torch.empty(shape, dtype=torch.float16 if f16 else torch.int32, device="cuda")
            return dev(A), dev(Bm), C, B.gemm_problem(batch, M, N, K, inst.group_m, inst.split_k)
        ops, byts = workloads.gemm_work(M, N, K, 2 if f16 else 1, 2 if f16 else 4, batch)
        W[name] = dict(inst=inst, build=build, ops=ops, bytes=byts, f16=f16,
                       text="%s batch=%d M=%d N=%d K=%d" % ("gemm_f16" if f16 else "gemm_u8s8", batch, M, N, K))

    add_gemm("gemm_u8s8_8192", 8192, 8192, 8192, False)
    add_gemm("gemm_f16_8192", 8192, 8192, 8192, True)
    add_gemm("gemm_f16_4096", 4096, 4096, 4096, True)
    add_gemm("bmm_f16_qk", 512, 64, 512, True, 192, lambda: workloads.bmm_qk_inputs(192, 512, 64, 512))
    add_gemm("bmm_f16_pv", 512, 512, 64, True, 192, lambda: workloads.bmm_pv_inputs(192, 512, 512, 64))

    def add_conv(name, f16):
        inst = tuned.load(name)

        def build():
            gen = workloads.conv2d_inputs if f16 else workloads.conv2d_u8s8_inputs
            X, Wt = gen(32, 56, 56, 64, 64, 3, 3, seed=3 if f16 else 6)
            Y = torch.empty((32, 56, 56, 64), dtype=torch.float16 if f16 else torch.int32, device="cuda")
            return dev(X), dev(Wt), Y, B.conv2d_problem(32, 56, 56, 64, 64, 3, 3, 1, 1, 1, inst.group_m, inst.split_k)
        ops, byts = workloads.conv_work(32, 56, 56, 64, 64, 3, 3, 1, 1, 1, in_bytes=2 if f16 else 1, out_bytes=2 if f16 else 4)
        W[name] = dict(inst=inst, build=build, ops=ops, bytes=byts, f16=f16,
                       text="conv2d_nhwc_%s N=32 H=W=56 C=64 K=64 3x3 s1 p1" % ("f16" if f16 else "u8s8"))

    add_conv("conv2d_f16_resnet", True)
    add_conv("conv2d_u8s8_resnet", False)
    return W


def settle(torch, mod, prob, a, b, c, stream, min_ms=200.0, max_ms=4000.0):
    """Untimed clock / power warm-up with the kernel that is about to be timed: at least ``min_ms`` of launches, then
    20-launch groups until two consecutive ones agree within 2 %.  Returns (milliseconds spent, last group's ms per
    launch)."""
    t0 = time.perf_counter()
    prev, spent = None, 0.0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    while True:
        e0.record()
        mod.launch_repeat(prob, a, b, c, 20, stream)
        e1.record()
        e1.synchronize()
        cur = e0.elapsed_time(e1) / 20.0
        spent = (time.perf_counter() - t0) * 1e3
        if spent >= min_ms and prev is not None and abs(cur - prev) <= 0.02 * prev:
            return spent, cur
        if spent >= max_ms:
            return spent, cur
        prev = cur


def measure(torch, B, w, steps, warmup, keep_rows=0, cold=False):
    """One workload: returns dict(wall_s, kernel_s, settle_ms, info[, cold_s][, rows])."""
    inst = w["inst"]
    mod = B.Module(inst.desc)
    a, b, c, prob = w["build"]()
    mod.bind_workspace(prob)
    stream = torch.cuda.current_stream().cuda_stream
    pa, pb, pc = a.data_ptr(), b.data_ptr(), c.data_ptr()
    spent, _ = settle(torch, mod, prob, pa, pb, pc, stream)
    if warmup > 0:
        mod.launch_repeat(prob, pa, pb, pc, warmup, stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()                                   # events on the launch stream (torch's current stream)
    mod.launch_repeat(prob, pa, pb, pc, steps, stream)     # exactly `steps` launches
    e1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    out = {"wall_s": wall, "kernel_s": e0.elapsed_time(e1) * 1e-3 / steps, "settle_ms": spent, "info": dict(mod.info)}
    if keep_rows:                                 # rows of the very buffer that was timed (the floor probe below reuses it)
        out["rows"] = c.reshape(-1, c.shape[-1])[:keep_rows].cpu().numpy()
    if inst.desc.colsum:
        # the column sums of B were made once (first launch above); what that pass costs when it is counted in
        torch.cuda.synchronize()
        e0.record()
        for _ in range(20):
            B.colsum_s8(pb, int(prob.bsum), int(prob.batch), int(prob.n), int(prob.k), int(prob.ldb),
                        int(prob.stride_b) if prob.op == B.HRN_OP_GEMM else 0, stream)
        e1.record()
        e1.synchronize()
        out["colsum_pass_s"] = e0.elapsed_time(e1) * 1e-3 / 20
    if cold:
        flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        costs = mod.time_cold(prob, pa, pb, pc, flush.data_ptr(), flush.numel(), repeat=9, stream=stream)
        out["cold_s"] = sorted(costs)[len(costs) // 2]
        # the floor of that launch: nothing but the algorithmic traffic, same flush, one dispatch
        rd = (a.numel() * a.element_size() + b.numel() * b.element_size() + 15) // 16 * 16
        wr = (c.numel() * c.element_size() + 15) // 16 * 16
        src = torch.empty(rd, dtype=torch.uint8, device="cuda")
        floor = B.probe_traffic_cold(src.data_ptr(), rd, pc, wr, flush.data_ptr(), flush.numel(), repeat=9, stream=stream)
        out["floor_s"] = sorted(floor)[len(floor) // 2] * 1e-6
        del flush, src
    mod.close()
    del a, b, c
    return out


def traffic_table():
    """instance -> measured HBM bytes per launch, from the tracked rocprofv3 counter runs (profiles/traffic.json)."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def measured_traffic(table, name, inst):
    """Bytes per launch when the profiled instance is the one that runs now, else None."""
    row = table.get(name)
    if not row or row.get("instance") != list(inst.desc.as_tuple()):
        return None
    return row.get("bytes")


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
        "hbm_read_1GiB_GBs": B.probe_read(src.data_ptr(), n, 10, st),
        "empty_kernel_256wg_us_per_launch": B.probe_launch(256, 2000, st),
        "empty_kernel_2048wg_us_per_launch": B.probe_launch(2048, 2000, st),
    }
    del src, dst
    # the vendor library on the same random operands, for orientation only; a library problem must not cost the line
    try:
        n = 8192
        a = (torch.randn(n, n, device="cuda") * 0.1).half()
        b = (torch.randn(n, n, device="cuda") * 0.1).half()
        for _ in range(20):
            torch.matmul(a, b.t())
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(50):
            torch.matmul(a, b.t())
        e1.record()
        torch.cuda.synchronize()
        out["vendor_library_gemm_f16_8192_TFLOPs"] = 2.0 * n ** 3 / (e0.elapsed_time(e1) * 1e-3 / 50) / 1e12
        del a, b
        a = torch.randint(-128, 128, (n, n), device="cuda", dtype=torch.int8)
        b = torch.randint(-128, 128, (n, n), device="cuda", dtype=torch.int8)
        for _ in range(20):
            torch._int_mm(a, b.t())
        torch.cuda.synchronize()
        e0.record()
        for _ in range(50):
            torch._int_mm(a, b.t())
        e1.record()
        torch.cuda.synchronize()
        out["vendor_library_gemm_s8s8_8192_TOPs"] = 2.0 * n ** 3 / (e0.elapsed_time(e1) * 1e-3 / 50) / 1e12
        del a, b
    except Exception as e:  # noqa: BLE001
        out["vendor_library_error"] = repr(e)[:200]
    return out


def run_prestage(torch, B, reps=200, cold_reps=10):
    """The library's own passes around the kernel, each timed warm (``reps`` back-to-back launches between two events)
    and cold (single launches, each after 1 GiB was streamed through the caches), with the algorithmic bytes it moves and
    the cold floor of exactly that traffic (``hrn_probe_traffic_cold``)."""
    from heron_amd import instances
    stream = torch.cuda.current_stream().cuda_stream
    flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rows = []

    def timed(name, shape, launch, read_bytes, write_bytes):
        for _ in range(10):
            launch()
        e0.record()
        for _ in range(reps):
            launch()
        e1.record()
        e1.synchronize()
        warm_us = e0.elapsed_time(e1) * 1e3 / reps
        cold = []
        for _ in range(cold_reps):
            flush.add_(1)
            e0.record()
            launch()
            e1.record()
            e1.synchronize()
            cold.append(e0.elapsed_time(e1) * 1e3)
        rb, wb = read_bytes - read_bytes % 16, write_bytes - write_bytes % 16
        psrc = torch.zeros(rb, dtype=torch.uint8, device="cuda")            # buffers of exactly the sizes the probe touches
        pdst = torch.empty(wb, dtype=torch.uint8, device="cuda")
        floor = B.probe_traffic_cold(psrc.data_ptr(), rb, pdst.data_ptr(), wb, flush.data_ptr(), flush.numel(), 5, stream)
        del psrc, pdst
        cold_us, floor_us = float(sorted(cold)[len(cold) // 2]), float(sorted(floor)[len(floor) // 2])
        rows.append({"pass": name, "shape": shape, "read_bytes": read_bytes, "write_bytes": write_bytes,
                     "warm_us": warm_us, "cold_us": cold_us, "floor_us_cold": floor_us,
                     "warm_GBs": (read_bytes + write_bytes) / warm_us / 1e3,
                     "cold_GBs": (read_bytes + write_bytes) / cold_us / 1e3})

    # NCW -> NWC activation of the conv1d sweep cases: 16 x 512 channels x 892 positions, fp16
    src = torch.randn(16, 512, 892, device="cuda").half()
    dst = torch.empty(16, 892, 512, dtype=torch.float16, device="cuda")
    timed("hrn_transpose_pad", "16 x (512 x 892) fp16 -> 16 x (892 x 512)",
          lambda: B.transpose_pad(src.data_ptr(), dst.data_ptr(), 16, 512, 892, 512, 2, stream),
          src.numel() * 2, dst.numel() * 2)
    # 3-channel stem -> 8 channels: 16 x 224 x 224 pixels, fp16
    src2 = torch.randn(16 * 224 * 224, 3, device="cuda").half()
    dst2 = torch.empty(16 * 224 * 224, 8, dtype=torch.float16, device="cuda")
    timed("hrn_pad_rows", "802816 pixels x 3 -> 8 channels fp16",
          lambda: B.pad_rows(src2.data_ptr(), dst2.data_ptr(), 16 * 224 * 224, 3, 8, 2, stream),
          src2.numel() * 2, dst2.numel() * 2)
    # stride-2 expansion of the transposed conv (16 x 56 x 56 x 64 fp16, channels last -> 111 x 111 with zeros between)
    src4 = torch.randn(16, 56, 56, 64, device="cuda").half()
    dst4 = torch.empty(16, 111, 111, 64, dtype=torch.float16, device="cuda")
    g4 = B.make_gather(2, (16, 111, 111, 64), [(16, 56 * 56 * 64, {0: 1}), (56, 56 * 64, {1: 1}, 0, 2),
                                               (56, 64, {2: 1}, 0, 2), (64, 1, {3: 1})])
    timed("hrn_gather_nd", "16 x 56 x 56 x 64 fp16 -> 16 x 111 x 111 x 64 (stride-2 zero expansion)",
          lambda: B.gather_nd(g4, src4.data_ptr(), dst4.data_ptr(), None, stream), src4.numel() * 2, dst4.numel() * 2)
    # column sums of the int8 weight operand of the 8192^3 GEMM
    src3 = torch.randint(-128, 128, (8192, 8192), dtype=torch.int8, device="cuda")
    dst3 = torch.empty(8192, dtype=torch.int32, device="cuda")
    timed("hrn_colsum_s8", "8192 x 8192 int8 -> 8192 int32",
          lambda: B.colsum_s8(src3.data_ptr(), dst3.data_ptr(), 1, 8192, 8192, stream=stream),
          src3.numel(), dst3.numel() * 4)
    # split-K: ResNet-50's 7x7x512 3x3 layer as a GEMM (M = 16*7*7, K = 9*512), 4 slices -> kernel + splitk_reduce_kernel
    desc = [d for d in instances.splitk_descs() if d.op == instances.GEMM and d.dtype == instances.F16][0]
    mod = B.Module(desc)
    M, K, N, split = 784, 4608, 512, 4
    a = (torch.randn(M, K, device="cuda") * 0.1).half()
    b = (torch.randn(N, K, device="cuda") * 0.1).half()
    c = torch.empty(M, N, dtype=torch.float16, device="cuda")
    prob = B.gemm_problem(1, M, N, K, 8, split_k=split)
    ws = B.splitk_workspace_bytes(desc, prob)
    timed("split-K GEMM + splitk_reduce_kernel", "784 x 4608 x 512 fp16, 4 slices (workspace %d bytes)" % ws,
          lambda: mod.launch(prob, a.data_ptr(), b.data_ptr(), c.data_ptr(), stream),
          (M * K + N * K) * 2 + ws, M * N * 2 + ws)
    mod.close()
    return rows


def roofline(w, seconds, workloads):
    """Roofline entry from the algorithmic work / bytes of one launch and its duration."""
    ai = w["ops"] / w["bytes"]
    peak_mfma = workloads.PEAK_FP16_TFLOPS if w["f16"] else workloads.PEAK_INT8_TOPS
    ridge = peak_mfma * 1e12 / (workloads.PEAK_HBM_GBS * 1e9)
    if ai >= ridge:
        ach = w["ops"] / seconds / 1e12
        return {"bound": "mfma", "achieved": ach, "peak": peak_mfma, "unit": "TFLOP/s" if w["f16"] else "TOP/s",
                "frac": ach / peak_mfma, "traffic": None}
    ach = w["bytes"] / seconds / 1e9
    return {"bound": "hbm", "achieved": ach, "peak": workloads.PEAK_HBM_GBS, "unit": "GB/s",
            "frac": ach / workloads.PEAK_HBM_GBS, "traffic": None}


def is_hbm_bound(w, workloads):
    peak_mfma = workloads.PEAK_FP16_TFLOPS if w["f16"] else workloads.PEAK_INT8_TOPS
    return w["ops"] / w["bytes"] < peak_mfma * 1e12 / (workloads.PEAK_HBM_GBS * 1e9)


def cpu_baseline(workloads, gpu_rows=None):
    """The CPU oracle's DL Boost-style GEMM on the 8192^3 problem (checker code used as a reported baseline only);
    the first rows of the GPU output of the timed buffers are checked against the same result."""
    import numpy as np
    import oracle
    cores = len(os.sched_getaffinity(0))
    M = K = N = 8192
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
    ref = oracle.gemm_u8s8s32_dlboost(A[:rows], Bm)
    dt = time.perf_counter() - t0
    out = {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TOP/s", "cores": oracle.num_threads(), "kind": "port",
           "sample": "%d rows of the 8192^3 u8s8 GEMM, scalar fallback (no AVX512-VNNI)" % rows}
    if gpu_rows is not None:
        out["gpu_rows_bit_exact"] = bool(np.array_equal(gpu_rows[:rows], ref[:len(gpu_rows)]))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE)
    ap.add_argument("--only", action="store_true", help="skip the 'also' workloads, the probes and the CPU baseline")
    ap.add_argument("--probe", action="store_true", help="only run the roofline probes (MFMA loop, 1 GiB copy)")
    ap.add_argument("--prestage", action="store_true",
                    help="only time the library's passes around the kernel (transpose, channel padding, column sums, "
                         "split-K reduction), warm and cold")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the hot path is a single-GPU kernel and no multi-GPU figure is produced "
              "(got --gpus %d)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from heron_amd import backend as B
    from heron_amd import tuned, workloads
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    B.lib()
    if args.probe:
        print(json.dumps({"probes": run_probes(torch, B)}))
        return
    if args.prestage:
        print(json.dumps({"prestage": run_prestage(torch, B)}))
        return
    if args.workload not in tuned.CASES:
        print("unknown workload %s (have %s)" % (args.workload, sorted(tuned.CASES)), file=sys.stderr)
        sys.exit(2)
    W = make_workloads(torch, workloads, tuned)
    table = traffic_table()

    w = W[args.workload]
    inst = w["inst"]
    check = args.workload == HEADLINE and not args.only
    hbm = is_hbm_bound(w, workloads)
    r = measure(torch, B, w, args.steps, args.warmup, keep_rows=64 if check else 0, cold=True)
    roof = roofline(w, r["cold_s"] if hbm else r["kernel_s"], workloads)
    roof["traffic"] = measured_traffic(table, args.workload, inst)
    line = {
        "metric": "%s throughput per GPU (tuned MFMA template)" % ("fp16 GEMM TFLOPS" if w["f16"] else "u8s8 GEMM TOPS"),
        "value": w["ops"] / r["wall_s"] / 1e12,
        "unit": "TFLOP/s" if w["f16"] else "TOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["wall_s"] * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if w["f16"] else "u8",
        "data": "synthetic",
        "config": {"workload": w["text"], "instance": repr(inst.desc), "record": inst.code,
                   "records_file": os.path.relpath(inst.records, ROOT), "group_m": inst.group_m, "split_k": inst.split_k,
                   "kernel_ms": r["kernel_s"] * 1e3, "clock_settle_ms": r["settle_ms"], "resources": r["info"]},
        "roofline": roof,
    }
    line["config"]["kernel_ms_cold"] = r["cold_s"] * 1e3       # single launches, each after 1 GiB went through the caches
    line["config"]["floor_us_cold"] = r["floor_s"] * 1e6
    if hbm:
        line["roofline"]["frac_of_floor"] = r["floor_s"] / r["cold_s"]
    if "colsum_pass_s" in r:
        line["config"]["weights"] = ("column sums of B prepared once with the weights (hrn_colsum_s8), outside the timed "
                                     "region, like the reference's pre-packed weight operand (ops/x86/dense.py:7-9)")
        line["config"]["colsum_pass_ms"] = r["colsum_pass_s"] * 1e3
        line["with_colsum_pass"] = {"ms_per_step": (r["wall_s"] + r["colsum_pass_s"]) * 1e3,
                                    "value": w["ops"] / (r["wall_s"] + r["colsum_pass_s"]) / 1e12}
    stable = {args.workload: w["ops"] / r["wall_s"] / 1e12}
    if not args.only:
        line["peaks"] = {"published": {"mfma_f16_TFLOPs": workloads.PEAK_FP16_TFLOPS, "mfma_i8_TOPs": workloads.PEAK_INT8_TOPS,
                                       "hbm_GBs": workloads.PEAK_HBM_GBS}, "used": "published"}
        try:
            line["peaks"]["measured"] = run_probes(torch, B)
        except Exception as e:  # noqa: BLE001 - context figures only
            line["peaks"]["measured"] = {"error": repr(e)[:200]}
        also = []
        for name, ww in W.items():
            if name == args.workload:
                continue
            steps = max(10, min(args.steps, 200))
            hbm = is_hbm_bound(ww, workloads)
            try:
                rr = measure(torch, B, ww, steps, min(args.warmup, 5), cold=True)
            except Exception as err:  # noqa: BLE001 - one side workload must not cost the headline
                also.append({"workload": ww["text"], "error": repr(err)[:200]})
                continue
            rf = roofline(ww, rr["cold_s"] if hbm else rr["kernel_s"], workloads)
            rf["traffic"] = measured_traffic(table, name, ww["inst"])
            peak = workloads.PEAK_FP16_TFLOPS if ww["f16"] else workloads.PEAK_INT8_TOPS
            row = {"workload": ww["text"], "value": ww["ops"] / rr["wall_s"] / 1e12,
                   "unit": "TFLOP/s" if ww["f16"] else "TOP/s", "steps": steps, "kernel_ms": rr["kernel_s"] * 1e3,
                   "record": ww["inst"].code, "instance": list(ww["inst"].desc.as_tuple()),
                   "frac_of_mfma_peak": ww["ops"] / rr["kernel_s"] / 1e12 / peak, "roofline": rf}
            row["kernel_ms_cold"] = rr["cold_s"] * 1e3
            row["floor_us_cold"] = rr["floor_s"] * 1e6
            if hbm:
                rf["frac_of_floor"] = rr["floor_s"] / rr["cold_s"]
                row["roofline_timed"] = "cold: every launch after 1 GiB was streamed through the caches"
            if "colsum_pass_s" in rr:
                row["colsum_pass_ms"] = rr["colsum_pass_s"] * 1e3
            stable[name] = row["value"]
            also.append(row)
        line["also"] = also
        try:
            line["cpu_baseline"] = cpu_baseline(workloads, r.get("rows") if args.workload == HEADLINE else None)
        except Exception as e:  # noqa: BLE001 - the GPU figures above are still worth printing
            line["cpu_baseline"] = {"value": None, "unit": None, "cores": 0, "kind": "port", "sample": "failed: %r" % (e,)}
    # fixed names for the three GEMM figures, whichever of them is the headline (the headline was the fp16 4096^3
    # GEMM in the first revision of this file and is the u8s8 8192^3 GEMM since)
    line["stable"] = {"gemm_f16_4096_TFLOPs": stable.get("gemm_f16_4096"), "gemm_f16_8192_TFLOPs": stable.get("gemm_f16_8192"),
                      "gemm_u8s8_8192_TOPs": stable.get("gemm_u8s8_8192")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
