"""HIP builder and measurer.

Counterparts of autotvm's LocalBuilder and the reference's LocalRunner / my_run_through_rpc
(runner/measure_methods.py:5-54,106-188):

* ``HipBuilder.build`` instantiates every sample (``task.instantiate``) and compiles the template
  instances in a pool of worker processes that never touch the GPU (``hrn_compile`` runs hipcc),
  honouring ``build_timeout``.
* ``HipRunner.run`` hands each built instance to a *measurement server*: one child process that
  owns the HIP context (as the reference times kernels behind a local RPC session).  The tuning
  process itself never initialises HIP, so its fork-based sampling stays safe, and a launch that
  exceeds ``timeout`` costs only the server, which is restarted (-> RUN_TIMEOUT).
  Timing has ``time_evaluator`` semantics (``hrn_time``); with more than two repeats the median is
  kept (measure_methods.py:167-171); with a verify function armed the output is compared with
  ``np.allclose(expected, out, rtol)`` and a mismatch is reported as error 100 (173-177).
"""
import multiprocessing as mp
import os
import time
import traceback
from concurrent.futures import ProcessPoolExecutor
from concurrent.futures import TimeoutError as FutureTimeout

import numpy as np

from .measure import BuildResult, MeasureErrorNo, MeasureResult

_spawn = mp.get_context("spawn")


def _problem_to_dict(p):
    """The shape fields of an hrn_problem; a split-K workspace and column sums are device memory of the process that
    launches, so the measurement server binds its own."""
    return {name: int(getattr(p, name)) for name, _ in p._fields_ if name not in ("workspace", "workspace_bytes", "bsum")}


def _compile_worker(desc_tuple, timeout_s):
    from .. import backend as B
    t0 = time.time()
    try:
        B.compile_desc(B.make_desc(*desc_tuple), timeout_s)
        return None, time.time() - t0
    except B.HeronRocmError as e:
        return (e.code, str(e)), time.time() - t0


class HipBuilder:
    def __init__(self, timeout=50, n_parallel=None):
        self.timeout = timeout
        self.n_parallel = n_parallel or min(16, os.cpu_count() or 1)
        self.task = None
        self.build_kwargs = None
        self._pool = None

    def set_task(self, task, build_kwargs=None):
        self.task = task
        self.build_kwargs = build_kwargs

    def _executor(self):
        if self._pool is None:
            self._pool = ProcessPoolExecutor(max_workers=self.n_parallel, mp_context=_spawn)
        return self._pool

    def build(self, measure_inputs):
        prepared = []
        for inp in measure_inputs:
            t0 = time.time()
            try:
                s, args = inp.task.instantiate(inp.config)
                desc = s.to_desc()
                arg_info = [(tuple(t.shape), t.dtype) for t in args]
                adapter = dict(s.info) if s.info.get('adapter', 'identity') != 'identity' else None
                prepared.append((desc.as_tuple(), _problem_to_dict(s.to_problem()), arg_info, None, t0, adapter))
            except Exception as e:  # noqa: BLE001 - reported as an instantiation error
                prepared.append((None, None, None, (MeasureErrorNo.INSTANTIATION_ERROR, repr(e)), t0, None))
        ex = self._executor()
        futures = {}
        for tup, _, _, err, _, _ in prepared:
            if err is None and tup not in futures:
                futures[tup] = ex.submit(_compile_worker, tup, float(self.timeout))
        results = []
        for tup, prob, arg_info, err, t0, adapter in prepared:
            if err is None:
                try:
                    cerr, _ = futures[tup].result(timeout=self.timeout + 30)
                except FutureTimeout:
                    cerr = (-5, "build timed out")
                except Exception as e:  # noqa: BLE001 - a dead worker
                    cerr = (-2, repr(e))
                if cerr is not None:
                    code = MeasureErrorNo.BUILD_TIMEOUT if cerr[0] == -5 else (
                        MeasureErrorNo.INSTANTIATION_ERROR if cerr[0] == -1 else MeasureErrorNo.COMPILE_DEVICE)
                    err = (code, cerr[1])
            results.append(BuildResult(tup, prob, arg_info, err, time.time() - t0, adapter))
        return results

    def close(self):
        if self._pool is not None:
            self._pool.shutdown(wait=False, cancel_futures=True)
            self._pool = None

    def __del__(self):
        try:
            self.close()
        except Exception:  # noqa: BLE001
            pass


LocalBuilder = HipBuilder


# ------------------------------------------------------------------------------ server side
_TORCH_DT = {"float16": "float16", "uint8": "uint8", "int8": "int8", "int32": "int32"}


def _operator_inputs(torch, info, ref_input):
    """Device tensors in the operator's own layouts: the reference inputs when given, random data otherwise.  The
    shapes must be the ones the operator declares (a mismatch would let the kernel read past an allocation)."""
    f16 = info['kind'] == 'f16'
    names = [n for n in info['reference_args'] if n != 'out']
    shapes = [tuple(int(x) for x in info['reference_args'][n]) for n in names]
    if ref_input is not None:                      # every shape is checked before anything is uploaded
        if len(ref_input) < len(names):
            raise ValueError("reference inputs: %d given, operator takes %d" % (len(ref_input), len(names)))
        for i, shape in enumerate(shapes):
            if tuple(np.shape(ref_input[i])) != shape:
                raise ValueError("reference input %d has shape %s, the operator declares %s"
                                 % (i, tuple(np.shape(ref_input[i])), shape))
    inputs = []
    for i, shape in enumerate(shapes):
        want = torch.float16 if f16 else (torch.uint8 if i == 0 else torch.int8)
        if ref_input is not None:
            t = torch.from_numpy(np.ascontiguousarray(ref_input[i])).to(want).cuda()
        elif f16:
            t = (torch.rand(shape, device="cuda") * 2 - 1).half()
        elif i == 0:
            t = torch.randint(0, 256, shape, dtype=torch.uint8, device="cuda")
        else:
            t = torch.randint(-128, 128, shape, dtype=torch.int8, device="cuda")
        inputs.append(t)
    return inputs


def _time_operator(torch, mod, info, prob, number, repeat, min_repeat_ms, ref_input=None, flush=None):
    """(seconds per call, result of the last call) of the operator, time_evaluator style: activation pre-stage + kernel +
    result reorder (hostops.run_operator recorded as an OperatorPlan and replayed) - the same definition with and
    without a result check.  The constant operand (reordered
    filter, generated right-hand side) is prepared once outside the timed calls, as a caller with fixed weights does.
    With ``flush`` (a device buffer larger than the caches) every repeat is ONE call after the buffer was streamed
    through the caches."""
    from .. import hostops
    inputs = _operator_inputs(torch, info, ref_input)
    gm, sk = int(prob.get('group_m', 8)), int(prob.get('split_k', 0))
    weights = hostops.prepare_constant(info, inputs)
    try:
        # the passes and the launch recorded once and replayed: what a caller with preallocated buffers pays per call
        plan = hostops.OperatorPlan(mod, info, inputs, group_m=gm, split_k=sk, constant=weights)
        call = plan.run
    except RuntimeError:
        # an adapter that moves data outside the library's passes cannot be replayed: time the eager call
        def call():
            return hostops.run_operator(mod, info, inputs, group_m=gm, split_k=sk, constant=weights)

    out = call()                                                             # warm-up, surfaces launch errors
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    costs = []
    if flush is not None:
        half = flush.numel() // 2
        for _ in range(repeat):
            flush[half:2 * half].copy_(flush[:half])
            e0.record()
            out = call()
            e1.record()
            e1.synchronize()
            costs.append(e0.elapsed_time(e1) * 1e-3)
        return costs, out
    for _ in range(repeat):
        num = number
        while True:
            e0.record()
            for _i in range(num):
                out = call()
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1)
            if ms >= min_repeat_ms or num >= (1 << 16):
                costs.append(ms * 1e-3 / num)
                number = num
                break
            num = max(num + 1, int(min(65536.0, min_repeat_ms * 1.2 / max(ms / num, 1e-4) + 1)))
    return costs, out


def _matches(ref_output, out, rtol):
    ref = np.asarray(ref_output, dtype=np.float64)
    if tuple(ref.shape) != tuple(out.shape):
        return False
    return bool(np.allclose(ref, out.astype(np.float64), rtol=rtol, atol=rtol * float(np.abs(ref).max()) * 1e-2))


def _server_main(conn, device_id):
    """Runs in the child that owns the GPU: answers 'info' and 'measure' requests until 'quit'."""
    try:
        import torch
        from .. import backend as B
        torch.cuda.set_device(device_id)
        mods = {}
        flush = None
        conn.send(("ready", None))
    except Exception:  # noqa: BLE001
        conn.send(("error", traceback.format_exc()))
        return
    while True:
        try:
            req = conn.recv()
        except EOFError:
            return
        kind = req[0]
        if kind == "quit":
            return
        try:
            if kind == "info":
                conn.send(("ok", B.device_info(device_id)))
                continue
            _, desc_tuple, prob, arg_info, number, repeat, min_repeat_ms, ref_input, ref_output, rtol = req[:10]
            cold = len(req) > 10 and req[10]
            adapter = req[11] if len(req) > 11 else None
            if desc_tuple not in mods:
                if len(mods) > 64:
                    mods.pop(next(iter(mods))).close()
                mods[desc_tuple] = B.Module(B.make_desc(*desc_tuple))
            mod = mods[desc_tuple]
            p = B.Problem()
            for k, v in prob.items():
                setattr(p, k, v)
            if cold and flush is None:
                flush = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
            if adapter is not None:
                # the operator reaches the kernel through an operand adapter: time pre-stage + kernel + post-stage on
                # operands in the operator's own layouts (the reference inputs when the result is checked), so that
                # the record's latency is what a caller pays and the kernel never sees an operand of the wrong size
                costs, out = _time_operator(torch, mod, adapter, prob, number, repeat, min_repeat_ms, ref_input,
                                            flush if cold else None)
                errno = MeasureErrorNo.NO_ERROR
                if ref_output is not None and not _matches(ref_output, out.cpu().numpy(), rtol):
                    errno = MeasureErrorNo.VERIFY_FAILED
                conn.send(("ok", (costs, errno)))
                continue
            tensors = []
            for i, (shape, dtype) in enumerate(arg_info):
                tdt = getattr(torch, _TORCH_DT[dtype])
                if ref_input is not None and i < len(ref_input):
                    host = np.ascontiguousarray(ref_input[i])
                    if tuple(host.shape) != tuple(shape):
                        raise ValueError("reference input %d has shape %s, the kernel's operand is %s"
                                         % (i, tuple(host.shape), tuple(shape)))
                    t = torch.from_numpy(host).to(tdt).cuda()
                elif i == len(arg_info) - 1:
                    t = torch.empty(shape, dtype=tdt, device="cuda")
                elif dtype == "float16":
                    t = (torch.rand(shape, device="cuda") * 2 - 1).to(tdt)
                elif dtype == "uint8":
                    t = torch.randint(0, 256, shape, dtype=tdt, device="cuda")
                else:
                    t = torch.randint(-128, 128, shape, dtype=tdt, device="cuda")
                tensors.append(t)
            torch.cuda.synchronize()
            if cold:
                # every launch starts from flushed caches (the reference runner's enable_cpu_cache_flush, on the GPU)
                costs = mod.time_cold(p, tensors[0].data_ptr(), tensors[1].data_ptr(), tensors[-1].data_ptr(),
                                      flush.data_ptr(), flush.numel(), repeat, 0)
            else:
                costs = mod.time(p, tensors[0].data_ptr(), tensors[1].data_ptr(), tensors[-1].data_ptr(),
                                 number, repeat, min_repeat_ms, 0)
            errno = MeasureErrorNo.NO_ERROR
            if ref_output is not None:
                if not _matches(ref_output, tensors[-1].cpu().numpy(), rtol):
                    errno = MeasureErrorNo.VERIFY_FAILED
            conn.send(("ok", (costs, errno)))
        except Exception as e:  # noqa: BLE001 - reported to the tuning process
            conn.send(("fail", repr(e)[:2048]))


class HipRunner:
    def __init__(self, number=3, repeat=4, min_repeat_ms=0, timeout=50, cooldown_interval=0.0,
                 enable_cpu_cache_flush=False, device_id=0):
        self.number = number
        self.repeat = repeat
        self.min_repeat_ms = min_repeat_ms
        self.timeout = timeout
        self.cooldown_interval = cooldown_interval
        self.cache_flush = bool(enable_cpu_cache_flush)
        self.device_id = device_id
        self.task = None
        self._proc = None
        self._conn = None

    # --- server management -------------------------------------------------------------
    def _start(self):
        parent, child = _spawn.Pipe()
        self._proc = _spawn.Process(target=_server_main, args=(child, self.device_id), daemon=True)
        self._proc.start()
        child.close()
        self._conn = parent
        if not parent.poll(300):
            self._stop(kill=True)
            raise RuntimeError("measurement server did not start")
        status, payload = parent.recv()
        if status != "ready":
            self._stop(kill=True)
            raise RuntimeError("measurement server failed to start:\n%s" % payload)

    def _stop(self, kill=False):
        if self._proc is None:
            return
        try:
            if not kill:
                self._conn.send(("quit",))
                self._proc.join(5)
        except Exception:  # noqa: BLE001
            pass
        if self._proc.is_alive():
            self._proc.kill()
            self._proc.join(5)
        self._conn.close()
        self._proc = self._conn = None

    def _request(self, req, timeout):
        if self._proc is None or not self._proc.is_alive():
            self._start()
        self._conn.send(req)
        if not self._conn.poll(timeout):
            self._stop(kill=True)
            return ("timeout", None)
        try:
            return self._conn.recv()
        except EOFError:
            self._stop(kill=True)
            return ("fail", "measurement server died")

    # --- reference interface -----------------------------------------------------------
    def set_task(self, task):
        self.task = task
        if hasattr(task, "device_id") and task.device_id is not None:
            if task.device_id != self.device_id:
                self._stop()
                self.device_id = task.device_id
        return None

    def get_build_kwargs(self):
        """Device limits for the schedule context (the ``check_gpu`` dictionary of the reference)."""
        status, payload = self._request(("info",), 300)
        if status != "ok":
            raise RuntimeError("cannot query the GPU: %s" % (payload,))
        keys = ('lds_bytes_per_wg', 'max_threads_per_wg', 'wave_size', 'regs_per_simd_lane', 'simd_per_cu', 'cu_count')
        check = {k: int(payload[k]) for k in keys}
        check['arch'] = payload['arch']
        return {'check_gpu': check}

    def run(self, measure_inputs, build_results):
        results = []
        for inp, br in zip(measure_inputs, build_results):
            tic = time.time()
            if br.error is not None:
                results.append(MeasureResult((RuntimeError(br.error[1]),), br.error[0], br.time_cost, time.time()))
                continue
            task = inp.task
            verify = not task.not_verify_correctness
            req = ("measure", br.desc_tuple, br.problem, br.arg_info, self.number, self.repeat,
                   float(self.min_repeat_ms), task.ref_input if verify else None,
                   task.ref_output if verify else None, getattr(task, "rtol", 0.1), self.cache_flush,
                   getattr(br, "adapter", None))
            status, payload = self._request(req, self.timeout)
            tstamp = time.time()
            if status == "ok":
                costs, errno = payload
                if len(costs) > 2:            # use the median
                    costs = sorted(costs)[len(costs) // 2]
                results.append(MeasureResult(costs, errno, tstamp - tic + br.time_cost, tstamp))
            elif status == "timeout":
                results.append(MeasureResult((RuntimeError("run timed out"),), MeasureErrorNo.RUN_TIMEOUT,
                                             self.timeout, tstamp))
            else:
                results.append(MeasureResult((RuntimeError(str(payload)),), MeasureErrorNo.RUNTIME_DEVICE,
                                             tstamp - tic + br.time_cost, tstamp))
            if self.cooldown_interval:
                time.sleep(self.cooldown_interval)
        return results

    def time_instance(self, s, args, number=3, repeat=4, min_repeat_ms=500, cold=False):
        """Final timing of one instance, as tests/quick_start/*/run.py:52-62 of the reference does with
        time_evaluator; returns the mean seconds per launch."""
        from .. import backend as B
        B.compile_desc(s.to_desc(), 300.0)
        req = ("measure", s.to_desc().as_tuple(), _problem_to_dict(s.to_problem()),
               [(tuple(t.shape), t.dtype) for t in args], number, repeat, float(min_repeat_ms), None, None, 0.1, cold,
               dict(s.info) if s.info.get('adapter', 'identity') != 'identity' else None)
        status, payload = self._request(req, max(self.timeout, 120))
        if status != "ok":
            raise RuntimeError("timing failed: %s %s" % (status, payload))
        costs, _ = payload
        return float(np.mean(costs))

    def close(self):
        self._stop()

    def __del__(self):
        try:
            self._stop()
        except Exception:  # noqa: BLE001
            pass


LocalRunner = HipRunner
