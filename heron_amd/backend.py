"""ctypes binding of ``librocm_heron.so`` (the C ABI declared in ``include/heron_rocm.h``).

This is the only door to the kernels: there is no CPU fallback.  If the shared library is
missing or a launch is attempted without a GPU, the calls raise ``HeronRocmError``.
"""
import ctypes
import os
import subprocess
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(CSRC, "librocm_heron.so")
INCLUDE = os.path.join(os.path.dirname(_HERE), "include")

HRN_DT_F16, HRN_DT_U8S8 = 0, 1
HRN_OP_GEMM, HRN_OP_CONV2D = 0, 1
HRN_OK = 0
HRN_E_BADPARAM, HRN_E_BUILD, HRN_E_LOAD, HRN_E_LAUNCH, HRN_E_TIMEOUT, HRN_E_NODEVICE = -1, -2, -3, -4, -5, -6
STATIC_WORKSPACE_BYTES = 32 << 20      # HRN_STATIC_WORKSPACE_BYTES

# flags every HIP translation unit of this package is compiled with
HIPCC_FLAGS = ["--offload-arch=gfx950", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


class HeronRocmError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("hrn error %d: %s" % (code, msg))
        self.code = code


class DevInfo(ctypes.Structure):
    _fields_ = [("arch", ctypes.c_char * 64), ("name", ctypes.c_char * 128),
                ("cu_count", ctypes.c_int32), ("wave_size", ctypes.c_int32),
                ("lds_bytes_per_wg", ctypes.c_int32), ("max_threads_per_wg", ctypes.c_int32),
                ("clock_khz", ctypes.c_int32), ("mem_clock_khz", ctypes.c_int32),
                ("mem_bus_bits", ctypes.c_int32), ("l2_bytes", ctypes.c_int32),
                ("regs_per_simd_lane", ctypes.c_int32), ("simd_per_cu", ctypes.c_int32),
                ("hbm_bytes", ctypes.c_uint64)]

    def as_dict(self):
        d = {}
        for name, _ in self._fields_:
            v = getattr(self, name)
            d[name] = v.decode() if isinstance(v, bytes) else int(v)
        return d


GATHER_DIMS = 6
GATHER_COPY, GATHER_CENTER_SQUARE = 0, 1


class Gather(ctypes.Structure):
    """hrn_gather: the affine index map of one injective pre-stage pass."""
    _fields_ = [("ndim", ctypes.c_int32), ("nsrc", ctypes.c_int32), ("elem_bytes", ctypes.c_int32), ("op", ctypes.c_int32),
                ("reserved", ctypes.c_int32 * 2),
                ("dst_dim", ctypes.c_int64 * GATHER_DIMS), ("dst_stride", ctypes.c_int64 * GATHER_DIMS),
                ("dst_live", ctypes.c_int64 * GATHER_DIMS), ("src_dim", ctypes.c_int64 * GATHER_DIMS),
                ("src_stride", ctypes.c_int64 * GATHER_DIMS), ("add", ctypes.c_int64 * GATHER_DIMS),
                ("div", ctypes.c_int64 * GATHER_DIMS), ("mul", (ctypes.c_int64 * GATHER_DIMS) * GATHER_DIMS)]


class KernelDesc(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("op", ctypes.c_int32), ("bm", ctypes.c_int32), ("bn", ctypes.c_int32),
                ("bkb", ctypes.c_int32), ("wm", ctypes.c_int32), ("wn", ctypes.c_int32), ("mfma", ctypes.c_int32),
                ("stages", ctypes.c_int32), ("swizzle", ctypes.c_int32), ("epilogue", ctypes.c_int32),
                ("waves_per_eu", ctypes.c_int32), ("conv_window", ctypes.c_int32), ("persistent", ctypes.c_int32),
                ("split_k", ctypes.c_int32), ("sched", ctypes.c_int32),
                ("load_spread", ctypes.c_int32), ("colsum", ctypes.c_int32), ("nt_store", ctypes.c_int32)]

    KEYS = ("dtype", "op", "bm", "bn", "bkb", "wm", "wn", "mfma", "stages", "swizzle", "epilogue", "waves_per_eu",
            "conv_window", "persistent", "split_k", "sched", "load_spread", "colsum", "nt_store")

    def as_tuple(self):
        return tuple(int(getattr(self, k)) for k in self.KEYS)

    def __repr__(self):
        return "KernelDesc(%s)" % ", ".join("%s=%d" % (k, getattr(self, k)) for k in self.KEYS)


class KernelInfo(ctypes.Structure):
    _fields_ = [("vgprs", ctypes.c_int32), ("agprs", ctypes.c_int32), ("sgprs", ctypes.c_int32),
                ("lds_bytes", ctypes.c_int32), ("scratch_bytes", ctypes.c_int32), ("occupancy", ctypes.c_int32),
                ("threads", ctypes.c_int32), ("reserved", ctypes.c_int32)]

    def as_dict(self):
        return {n: int(getattr(self, n)) for n, _ in self._fields_ if n != "reserved"}


class Problem(ctypes.Structure):
    _fields_ = [("op", ctypes.c_int32), ("batch", ctypes.c_int32),
                ("m", ctypes.c_int32), ("n", ctypes.c_int32), ("k", ctypes.c_int32),
                ("lda", ctypes.c_int32), ("ldb", ctypes.c_int32), ("ldc", ctypes.c_int32),
                ("stride_a", ctypes.c_int64), ("stride_b", ctypes.c_int64), ("stride_c", ctypes.c_int64),
                ("cn", ctypes.c_int32), ("ch", ctypes.c_int32), ("cw", ctypes.c_int32), ("ci", ctypes.c_int32),
                ("co", ctypes.c_int32), ("kh", ctypes.c_int32), ("kw", ctypes.c_int32),
                ("cstride", ctypes.c_int32), ("cpad", ctypes.c_int32), ("cdil", ctypes.c_int32),
                ("group_m", ctypes.c_int32),
                ("cstride_w", ctypes.c_int32), ("cpad_w", ctypes.c_int32), ("cdil_w", ctypes.c_int32),
                ("split_k", ctypes.c_int32), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_size_t),
                ("bsum", ctypes.c_void_p)]


def make_desc(dtype, op=HRN_OP_GEMM, bm=128, bn=128, bkb=128, wm=2, wn=2, mfma=32, stages=2, swizzle=1,
              epilogue=0, waves_per_eu=0, conv_window=0, persistent=0, split_k=0, sched=1, load_spread=2, colsum=0, nt_store=0):
    d = KernelDesc()
    d.colsum = colsum
    d.nt_store = nt_store
    d.conv_window, d.persistent, d.split_k, d.sched, d.load_spread = conv_window, persistent, split_k, sched, load_spread
    d.dtype, d.op, d.bm, d.bn, d.bkb, d.wm, d.wn = dtype, op, bm, bn, bkb, wm, wn
    d.mfma, d.stages, d.swizzle, d.epilogue, d.waves_per_eu = mfma, stages, swizzle, epilogue, waves_per_eu
    return d


def build_library(force=True, verbose=False):
    """Compile ``csrc/hrn_api.cpp`` into ``csrc/librocm_heron.so`` with hipcc (cross-compiles without a GPU)."""
    if os.path.exists(LIB_PATH) and not force:
        return LIB_PATH
    hipcc = os.environ.get("HRN_HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-O2", "-fPIC", "-shared"] + HIPCC_FLAGS + [os.path.join(CSRC, "hrn_api.cpp"), "-o", LIB_PATH + ".tmp"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building librocm_heron.so failed:\n" + r.stderr[-4000:])
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    if verbose:
        print("built", LIB_PATH)
    global _lib
    _lib = None
    return LIB_PATH


_lib = None
_lock = threading.Lock()

_vp, _i, _d = ctypes.c_void_p, ctypes.c_int, ctypes.c_double

# every symbol include/heron_rocm.h declares: name -> (restype, argtypes)
SYMBOLS = {
    "hrn_device_info": (_i, [_i, ctypes.POINTER(DevInfo)]),
    "hrn_check_desc": (_i, [ctypes.POINTER(KernelDesc)]),
    "hrn_compile": (_i, [ctypes.POINTER(KernelDesc), _d, ctypes.c_char_p, ctypes.c_size_t]),
    "hrn_build": (_i, [ctypes.POINTER(KernelDesc), _d, ctypes.POINTER(_vp)]),
    "hrn_module_info": (_i, [_vp, ctypes.POINTER(KernelInfo)]),
    "hrn_module_free": (None, [_vp]),
    "hrn_lds_bytes": (_i, [ctypes.POINTER(KernelDesc)]),
    "hrn_launch_gemm_f16": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_gemm_u8s8": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_bmm_f16": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_conv2d_nhwc_f16": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_bmm_u8s8": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_conv2d_nhwc_u8s8": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_splitk_static": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp]),
    "hrn_launch_repeat": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _i, _vp]),
    "hrn_time": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _i, _i, _d, ctypes.POINTER(_d), _vp]),
    "hrn_time_cold": (_i, [_vp, ctypes.POINTER(Problem), _vp, _vp, _vp, _vp, ctypes.c_size_t, _i, ctypes.POINTER(_d), _vp]),
    "hrn_splitk_workspace_bytes": (ctypes.c_int64, [ctypes.POINTER(KernelDesc), ctypes.POINTER(Problem)]),
    "hrn_problem_gemm": (None, [ctypes.POINTER(Problem), _i, _i, _i, _i]),
    "hrn_problem_conv2d": (None, [ctypes.POINTER(Problem)] + [_i] * 10),
    "hrn_problem_conv2d_hw": (None, [ctypes.POINTER(Problem)] + [_i] * 13),
    "hrn_probe_mfma": (_i, [_i, _i, _i, ctypes.POINTER(_d), _vp]),
    "hrn_probe_copy": (_i, [_vp, _vp, ctypes.c_size_t, _i, ctypes.POINTER(_d), _vp]),
    "hrn_probe_launch": (_i, [_i, _i, ctypes.POINTER(_d), _vp]),
    "hrn_pad_rows": (_i, [_vp, _vp, ctypes.c_size_t, _i, _i, _i, _vp]),
    "hrn_colsum_s8": (_i, [_vp, _vp, _i, _i, _i, _i, ctypes.c_int64, _vp]),
    "hrn_transpose_pad": (_i, [_vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "hrn_gather_nd": (_i, [ctypes.POINTER(Gather), _vp, _vp, _vp, _vp]),
    "hrn_probe_read": (_i, [_vp, ctypes.c_size_t, _i, ctypes.POINTER(_d), _vp]),
    "hrn_probe_traffic_cold": (_i, [_vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _i, ctypes.POINTER(_d), _vp]),
    "hrn_last_error": (ctypes.c_char_p, []),
    "hrn_version": (ctypes.c_char_p, []),
}


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise HeronRocmError(HRN_E_LOAD, "%s is missing: run __graft_entry__.build() "
                                     "(or heron_amd.backend.build_library())" % LIB_PATH)
            L = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in SYMBOLS.items():
                fn = getattr(L, name)
                fn.restype = res
                fn.argtypes = args
            _lib = L
    return _lib


def _check(rc):
    if rc != HRN_OK:
        raise HeronRocmError(rc, lib().hrn_last_error().decode(errors="replace"))


def device_info(device=0):
    info = DevInfo()
    _check(lib().hrn_device_info(device, ctypes.byref(info)))
    return info.as_dict()


def check_desc(desc):
    """True when the descriptor satisfies the template's structural constraints."""
    return lib().hrn_check_desc(ctypes.byref(desc)) == HRN_OK


def lds_bytes(desc):
    rc = lib().hrn_lds_bytes(ctypes.byref(desc))
    if rc < 0:
        _check(rc)
    return rc


def compile_desc(desc, timeout_s=0.0):
    """hipcc the instance into the cache (no GPU needed); returns the code object path."""
    buf = ctypes.create_string_buffer(4096)
    _check(lib().hrn_compile(ctypes.byref(desc), float(timeout_s), buf, 4096))
    return buf.value.decode()


def gemm_problem(batch, m, n, k, group_m=8, split_k=0):
    p = Problem()
    lib().hrn_problem_gemm(ctypes.byref(p), batch, m, n, k)
    p.group_m = group_m
    p.split_k = split_k
    return p


def splitk_workspace_bytes(desc, problem):
    """Bytes of device workspace a split-K launch of ``desc`` on ``problem`` needs (0 for other instances)."""
    n = lib().hrn_splitk_workspace_bytes(ctypes.byref(desc), ctypes.byref(problem))
    if n < 0:
        _check(int(n))
    return int(n)


def _pair(v):
    return (int(v), int(v)) if isinstance(v, int) else (int(v[0]), int(v[1]))


def conv2d_problem(n, h, w, ci, co, kh, kw, stride, pad, dil, group_m=8, split_k=0):
    """``stride``, ``pad`` and ``dil`` are ints or (height, width) pairs."""
    p = Problem()
    (sh, sw), (ph, pw), (dh, dw) = _pair(stride), _pair(pad), _pair(dil)
    lib().hrn_problem_conv2d_hw(ctypes.byref(p), n, h, w, ci, co, kh, kw, sh, sw, ph, pw, dh, dw)
    p.group_m = group_m
    p.split_k = split_k
    return p


def probe_mfma(dtype, mfma=32, random_operands=True, stream=0):
    """Dense T(FL)OP/s of a register-resident MFMA loop on all CUs (measured roofline denominator)."""
    out = _d()
    _check(lib().hrn_probe_mfma(dtype, mfma, 1 if random_operands else 0, ctypes.byref(out), stream))
    return out.value


def probe_launch(grid=256, repeat=2000, stream=0):
    """Microseconds per back-to-back dispatch of a kernel that does nothing."""
    out = ctypes.c_double()
    _check(lib().hrn_probe_launch(grid, repeat, ctypes.byref(out), stream))
    return out.value


def colsum_s8(b_ptr, out_ptr, batch, n, k, ldb=None, stride_b=None, stream=0):
    """out[b*n + j] = sum_k B[b][j][k] of an int8 operand (device pointers; out holds batch * n int32): the
    weight-side preparation of a ``colsum`` instance."""
    ldb = k if ldb is None else ldb
    stride_b = n * ldb if stride_b is None else stride_b
    _check(lib().hrn_colsum_s8(b_ptr, out_ptr, batch, n, k, ldb, stride_b, stream))


def pad_rows(src_ptr, dst_ptr, rows, c, cp, elem_bytes, stream=0):
    """Zero-pads rows of c elements to cp elements (device pointers, dst holds rows * cp elements)."""
    _check(lib().hrn_pad_rows(src_ptr, dst_ptr, rows, c, cp, elem_bytes, stream))


def transpose_pad(src_ptr, dst_ptr, batch, rows, cols, rows_padded, elem_bytes, stream=0):
    """dst[b][c][r] = src[b][r][c], rows of dst zero-padded to rows_padded (device pointers)."""
    _check(lib().hrn_transpose_pad(src_ptr, dst_ptr, batch, rows, cols, rows_padded, elem_bytes, stream))


def make_gather(elem_bytes, dst_dim, src, dst_stride=None, dst_live=None, op=GATHER_COPY):
    """Builds an hrn_gather.  ``dst_dim``: extents of dst (outermost first; contiguous unless ``dst_stride`` is given);
    ``src``: one entry per source coordinate, ``(extent, stride, {dst dimension: multiplier}, add, div)`` with ``add`` and
    ``div`` optional (0 and 1): coordinate = (add + sum multiplier * index) / div."""
    g = Gather()
    nd, ns = len(dst_dim), len(src)
    if not (1 <= nd <= GATHER_DIMS and 1 <= ns <= GATHER_DIMS):
        raise ValueError("a gather has 1..%d dst dimensions and source coordinates" % GATHER_DIMS)
    g.ndim, g.nsrc, g.elem_bytes, g.op = nd, ns, int(elem_bytes), int(op)
    stride = 1
    for d in range(nd - 1, -1, -1):
        g.dst_dim[d] = int(dst_dim[d])
        g.dst_stride[d] = int(dst_stride[d]) if dst_stride is not None else stride
        g.dst_live[d] = int(dst_live[d]) if dst_live is not None else int(dst_dim[d])
        stride *= int(dst_dim[d])
    for s, entry in enumerate(src):
        extent, sstride, muls = entry[0], entry[1], entry[2]
        g.src_dim[s], g.src_stride[s] = int(extent), int(sstride)
        g.add[s] = int(entry[3]) if len(entry) > 3 else 0
        g.div[s] = int(entry[4]) if len(entry) > 4 else 1
        for d, m in muls.items():
            g.mul[s][d] = int(m)
    return g


def gather_nd(g, src_ptr, dst_ptr, aux_ptr=None, stream=0):
    """dst = f(gather(src)) as one pass of the library (device pointers; see hrn_gather in the header)."""
    _check(lib().hrn_gather_nd(ctypes.byref(g), src_ptr, aux_ptr, dst_ptr, stream))


def probe_read(src_ptr, nbytes, repeat=10, stream=0):
    """GB/s of a read-only stream over device memory."""
    out = ctypes.c_double()
    _check(lib().hrn_probe_read(src_ptr, nbytes, repeat, ctypes.byref(out), stream))
    return out.value


def probe_traffic_cold(src_ptr, read_bytes, dst_ptr, write_bytes, flush_ptr, flush_bytes, repeat=5, stream=0):
    """Microseconds of ``repeat`` single cold launches of a kernel that only reads ``read_bytes`` and writes
    ``write_bytes``: the floor of a workload's cold launch (same flush as ``Module.time_cold``)."""
    out = (_d * repeat)()
    _check(lib().hrn_probe_traffic_cold(src_ptr, read_bytes, dst_ptr, write_bytes, flush_ptr, flush_bytes, repeat, out, stream))
    return list(out)


def probe_copy(src_ptr, dst_ptr, nbytes, repeat=10, stream=0):
    """GB/s (read + write) of a plain 16-byte-per-lane copy kernel over caller-owned device memory."""
    out = _d()
    _check(lib().hrn_probe_copy(src_ptr, dst_ptr, nbytes, repeat, ctypes.byref(out), stream))
    return out.value


class Module:
    """One loaded template instance (``hrn_module``)."""

    def __init__(self, desc, timeout_s=0.0):
        self.desc = desc
        h = _vp()
        _check(lib().hrn_build(ctypes.byref(desc), float(timeout_s), ctypes.byref(h)))
        self._h = h
        info = KernelInfo()
        _check(lib().hrn_module_info(self._h, ctypes.byref(info)))
        self.info = info.as_dict()

    def bind_workspace(self, problem):
        """Split-K instances: point ``problem`` at a device workspace owned by this module (torch supplies the
        memory; it grows on demand and is shared by the launches of this module, which therefore must not overlap)."""
        if not self.desc.split_k or problem.workspace:
            return problem
        if problem.split_k < 1:
            problem.split_k = 1
        need = splitk_workspace_bytes(self.desc, problem)
        ws = getattr(self, "_ws", None)
        if ws is None or ws.numel() < need:
            import torch
            self._ws = ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device="cuda")
        problem.workspace = ws.data_ptr()
        problem.workspace_bytes = ws.numel()
        return problem

    def bind_colsum(self, problem, b_ptr, stream=0):
        """Colsum instances: when the caller supplied no column sums of B (``problem.bsum``), compute them now into a
        buffer of this module - fresh on every call, since only the caller knows whether B has changed; callers with
        fixed weights compute them once (``colsum_s8``) and set ``problem.bsum`` themselves."""
        if not self.desc.colsum or problem.bsum:
            return problem
        need = int(problem.batch) * int(problem.n) * 4
        buf = getattr(self, "_bs", None)
        if buf is None or buf.numel() < need:
            import torch
            self._bs = buf = torch.empty(max(need, 4096), dtype=torch.uint8, device="cuda")
        colsum_s8(b_ptr, buf.data_ptr(), int(problem.batch), int(problem.n), int(problem.k), int(problem.ldb),
                  int(problem.stride_b) if problem.op == HRN_OP_GEMM else 0, stream)
        problem.bsum = buf.data_ptr()
        return problem

    def _launcher(self, problem):
        L = lib()
        if self.desc.op == HRN_OP_CONV2D:
            return L.hrn_launch_conv2d_nhwc_u8s8 if self.desc.dtype == HRN_DT_U8S8 else L.hrn_launch_conv2d_nhwc_f16
        if self.desc.dtype == HRN_DT_U8S8:
            return L.hrn_launch_bmm_u8s8 if problem.batch > 1 else L.hrn_launch_gemm_u8s8
        return L.hrn_launch_bmm_f16 if problem.batch > 1 else L.hrn_launch_gemm_f16

    def launch(self, problem, a_ptr, b_ptr, c_ptr, stream=0):
        self.bind_workspace(problem)
        self.bind_colsum(problem, b_ptr, stream)
        _check(self._launcher(problem)(self._h, ctypes.byref(problem), a_ptr, b_ptr, c_ptr, stream))

    def launch_splitk_static(self, problem, a_ptr, b_ptr, c_ptr, stream=0):
        """Split-K launch whose partial sums live in the library's own static device workspace (no allocation)."""
        _check(lib().hrn_launch_splitk_static(self._h, ctypes.byref(problem), a_ptr, b_ptr, c_ptr, stream))

    def launch_repeat(self, problem, a_ptr, b_ptr, c_ptr, count, stream=0):
        """``count`` back-to-back launches issued from one host call."""
        self.bind_workspace(problem)
        self.bind_colsum(problem, b_ptr, stream)
        _check(lib().hrn_launch_repeat(self._h, ctypes.byref(problem), a_ptr, b_ptr, c_ptr, count, stream))

    def time_cold(self, problem, a_ptr, b_ptr, c_ptr, flush_ptr, flush_bytes, repeat=4, stream=0):
        """Seconds of ``repeat`` single launches, each after the caches were flushed with the caller's buffer."""
        self.bind_workspace(problem)
        self.bind_colsum(problem, b_ptr, stream)
        costs = (_d * repeat)()
        _check(lib().hrn_time_cold(self._h, ctypes.byref(problem), a_ptr, b_ptr, c_ptr, flush_ptr, flush_bytes, repeat,
                                   costs, stream))
        return list(costs)

    def time(self, problem, a_ptr, b_ptr, c_ptr, number=3, repeat=4, min_repeat_ms=0.0, stream=0):
        """time_evaluator-style timing of the kernel.  For a colsum instance without ``problem.bsum`` the column
        sums of B are computed once before the timed launches (weights are fixed while a kernel is timed)."""
        self.bind_workspace(problem)
        self.bind_colsum(problem, b_ptr, stream)
        costs = (_d * repeat)()
        _check(lib().hrn_time(self._h, ctypes.byref(problem), a_ptr, b_ptr, c_ptr, number, repeat,
                              float(min_repeat_ms), costs, stream))
        return list(costs)

    def close(self):
        if getattr(self, "_h", None):
            lib().hrn_module_free(self._h)
            self._h = None
        self._ws = None
        self._bs = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
