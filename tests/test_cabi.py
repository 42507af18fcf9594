"""The C ABI library loads and exports every symbol include/heron_rocm.h declares (no GPU needed)."""
import ctypes
import os
import re

import numpy as np

from heron_amd import backend as B
from heron_amd import instances

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "heron_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hrn_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_exported_and_bound():
    names = declared_symbols()
    assert len(names) >= 16
    L = ctypes.CDLL(B.LIB_PATH)
    for n in names:
        assert hasattr(L, n), n
    assert set(names) == set(B.SYMBOLS), set(names) ^ set(B.SYMBOLS)
    assert b"gfx950" in B.lib().hrn_version()


def header_struct(name):
    """(field name, C type, array length) of every member of ``struct name`` in the header, in declaration order."""
    text = open(os.path.join(ROOT, "include", "heron_rocm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    macros = dict(re.findall(r"#define (HRN_\w+) (\d+)", text))
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
    out = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        ctype, names = re.match(r"((?:u?int\d+_t|size_t|char|(?:const\s+)?void\s*\*))\s*(.*)", decl, flags=re.S).groups()
        for n in names.split(","):
            m = re.match(r"\s*(\w+)((?:\[\w+\])*)\s*$", n)
            dims = [int(macros.get(x, x)) for x in re.findall(r"\[(\w+)\]", m.group(2))]
            out.append((m.group(1), ctype.replace(" ", ""), int(np.prod(dims)) if dims else 0))
    return out


C_TYPES = {"int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64, "uint64_t": ctypes.c_uint64, "size_t": ctypes.c_size_t,
           "void*": ctypes.c_void_p, "constvoid*": ctypes.c_void_p, "char": ctypes.c_char}


def test_struct_layouts_match_header():
    """Every ctypes structure has the header's members, in the header's order, with the header's types."""
    for name, cls in (("hrn_kernel_desc", B.KernelDesc), ("hrn_kernel_info", B.KernelInfo), ("hrn_problem", B.Problem),
                      ("hrn_devinfo", B.DevInfo), ("hrn_gather", B.Gather)):
        want = [(n, C_TYPES[t] * k if k else C_TYPES[t]) for n, t, k in header_struct(name)]
        have = [(n, t) for n, t in cls._fields_]
        assert [n for n, _ in have] == [n for n, _ in want], name
        for (n, th), (_, tw) in zip(have, want):
            def scalar(t):
                while hasattr(t, "_length_"):
                    t = t._type_                                     # element type of a (nested) array
                return t._type_
            assert ctypes.sizeof(th) == ctypes.sizeof(tw) and scalar(th) == scalar(tw), (name, n)
    assert ctypes.sizeof(B.KernelDesc) == 19 * 4
    assert B.KernelDesc.KEYS == tuple(n for n, _ in B.KernelDesc._fields_)


def test_check_desc_mirrors_template_constraints():
    ok = instances.D(instances.F16, instances.GEMM, 256, 256, 128, 2, 2, 32, 2, 2)
    assert B.check_desc(ok) and B.lds_bytes(ok) == 131072
    bad = [
        instances.D(instances.F16, instances.GEMM, 256, 256, 128, 2, 2, 32, 3, 2),    # 192 KiB LDS
        instances.D(instances.F16, instances.GEMM, 256, 128, 64, 4, 2, 16, 2, 3, epi=1, pers=1),   # persistent with one k-step per tile
        instances.D(instances.F16, instances.GEMM, 128, 128, 128, 2, 2, 32, 2, 1, epi=1, pers=1, split=1),   # persistent + split-K
        instances.D(instances.F16, instances.GEMM, 192, 128, 128, 3, 2, 32, 2, 1),    # wave rows not a power of two
        instances.D(instances.F16, instances.GEMM, 96, 128, 128, 2, 2, 32, 2, 0),     # 96 rows / (2 waves x 32)
        instances.D(instances.F16, instances.GEMM, 128, 128, 256, 2, 2, 16, 2, 2),    # swizzle period 32 > mfma 16
        instances.D(instances.F16, instances.GEMM, 128, 128, 128, 2, 2, 32, 2, 1, win=1),   # window mode is a conv load path
        instances.D(instances.F16, instances.GEMM, 512, 512, 64, 2, 2, 32, 2, 0),     # 1024 accumulators
        instances.D(instances.F16, instances.GEMM, 128, 128, 128, 8, 4, 32, 2, 0),    # 32 waves
    ]
    for d in bad:
        assert not B.check_desc(d), d
        assert B.lib().hrn_last_error()


def test_problem_helpers():
    p = B.gemm_problem(3, 100, 200, 64)
    assert (p.batch, p.m, p.n, p.k, p.lda, p.ldb, p.ldc, p.stride_c) == (3, 100, 200, 64, 64, 64, 200, 20000)
    c = B.conv2d_problem(32, 56, 56, 64, 64, 3, 3, 1, 1, 1)
    assert (c.m, c.n, c.k) == (32 * 56 * 56, 64, 576)
    c = B.conv2d_problem(1, 15, 15, 8, 16, 3, 3, 2, 1, 1)
    assert c.m == 8 * 8


def test_compile_without_gpu_and_shipped_instances_present():
    d = instances.BEST["small"]
    path = B.compile_desc(d, 120.0)
    assert path.endswith(".hsaco") and os.path.getsize(path) > 1000
    assert os.path.exists(path[:-6] + ".info")


def test_compile_error_paths(tmp_path, monkeypatch):
    """A path buffer that is too small, a compiler that fails and a compiler that outlives the limit are reported as
    errors with a message; nothing is left in the cache for them."""
    import stat
    d = instances.BEST["small"]
    L = B.lib()
    tiny = ctypes.create_string_buffer(8)
    assert L.hrn_compile(ctypes.byref(d), 120.0, tiny, 8) == -1 and b"too small" in L.hrn_last_error()
    assert L.hrn_compile(ctypes.byref(d), 120.0, None, 0) == 0
    monkeypatch.setenv("HRN_CACHE_DIR", str(tmp_path / "cache"))
    monkeypatch.setenv("HRN_HIPCC_FLAGS", "--no-such-flag")
    buf = ctypes.create_string_buffer(4096)
    assert L.hrn_compile(ctypes.byref(d), 120.0, buf, 4096) == -2 and b"hipcc failed" in L.hrn_last_error()
    monkeypatch.setenv("HRN_HIPCC_FLAGS", "")
    slow = tmp_path / "slow_cc.sh"
    slow.write_text("#!/bin/sh\nsleep 30\n")
    slow.chmod(slow.stat().st_mode | stat.S_IEXEC)
    monkeypatch.setenv("HRN_HIPCC", str(slow))
    assert L.hrn_compile(ctypes.byref(d), 0.5, buf, 4096) == -5 and b"exceeded" in L.hrn_last_error()
    assert not list((tmp_path / "cache").glob("*.hsaco"))


def test_prestage_entry_points_reject_bad_arguments_without_a_gpu():
    """Argument checks of the pre-stage kernels and probes run before any HIP call, so they can be exercised here."""
    L = B.lib()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.cast(buf, ctypes.c_void_p)
    assert L.hrn_pad_rows(p, p, 4, 3, 6, 2, None) == B.HRN_E_BADPARAM          # 12-byte rows are not whole 16-byte words
    assert b"pad_rows" in L.hrn_last_error()
    assert L.hrn_pad_rows(p, p, 4, 9, 8, 2, None) == B.HRN_E_BADPARAM          # padded row shorter than the row
    assert L.hrn_pad_rows(None, p, 4, 3, 8, 2, None) == B.HRN_E_BADPARAM
    assert L.hrn_pad_rows(p, p, 0, 3, 8, 2, None) == 0                          # nothing to do is not an error
    assert L.hrn_transpose_pad(p, p, 1, 8, 8, 4, 2, None) == B.HRN_E_BADPARAM   # fewer padded rows than rows
    assert L.hrn_transpose_pad(p, p, 1, 8, 8, 8, 3, None) == B.HRN_E_BADPARAM   # 3-byte elements
    assert L.hrn_transpose_pad(p, p, 70000, 8, 8, 8, 2, None) == B.HRN_E_BADPARAM
    assert L.hrn_transpose_pad(p, p, 0, 8, 8, 8, 2, None) == 0
    out = ctypes.c_double()
    assert L.hrn_probe_launch(0, 10, ctypes.byref(out), None) == B.HRN_E_BADPARAM
    assert L.hrn_probe_launch(256, 10, None, None) == B.HRN_E_BADPARAM
    assert L.hrn_probe_read(p, 24, 1, ctypes.byref(out), None) == B.HRN_E_BADPARAM   # not a multiple of 16 bytes


def test_gather_rejects_bad_maps_without_a_gpu():
    L = B.lib()
    buf = ctypes.create_string_buffer(256)
    p = ctypes.cast(buf, ctypes.c_void_p)
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})])
    assert (g.ndim, g.nsrc, g.dst_stride[0], g.dst_stride[1], g.dst_live[1], g.mul[0][0], g.mul[1][1], g.div[0]) == (2, 2, 8, 1, 8, 1, 1, 1)
    assert L.hrn_gather_nd(None, p, None, p, None) == B.HRN_E_BADPARAM
    g.dst_stride[1] = 2
    assert L.hrn_gather_nd(ctypes.byref(g), p, None, p, None) == B.HRN_E_BADPARAM and b"stride 1" in L.hrn_last_error()
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1}, 0, 0)])                    # divisor 0
    assert L.hrn_gather_nd(ctypes.byref(g), p, None, p, None) == B.HRN_E_BADPARAM and b"divisor" in L.hrn_last_error()
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})], dst_live=(4, 9))         # live beyond the extent
    assert L.hrn_gather_nd(ctypes.byref(g), p, None, p, None) == B.HRN_E_BADPARAM
    g = B.make_gather(2, (4, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})], op=B.GATHER_CENTER_SQUARE)   # no aux tensor
    assert L.hrn_gather_nd(ctypes.byref(g), p, None, p, None) == B.HRN_E_BADPARAM
    g = B.make_gather(2, (0, 8), [(4, 8, {0: 1}), (8, 1, {1: 1})])                          # nothing to do is not an error
    assert L.hrn_gather_nd(ctypes.byref(g), p, None, p, None) == 0
