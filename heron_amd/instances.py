"""Named template instances that ship pre-compiled (tests, smoke and the benchmark load these).

``precompile`` drives ``hrn_compile`` over a list of descriptors in worker processes; it needs
hipcc but no GPU, so it runs at build time and the code objects travel with the tree.
"""
import os
from concurrent.futures import ProcessPoolExecutor

from . import backend as B

F16, U8 = B.HRN_DT_F16, B.HRN_DT_U8S8
GEMM, CONV = B.HRN_OP_GEMM, B.HRN_OP_CONV2D


def D(dtype, op, bm, bn, bkb, wm, wn, mfma, stages, swz, epi=0, wpe=0, win=0, pers=0, split=0, sched=1, spread=2, colsum=0, nt=0):
    return B.make_desc(dtype, op, bm, bn, bkb, wm, wn, mfma, stages, swz, epi, wpe, win, pers, split, sched, spread, colsum, nt)


# (bm, bn, bkb, wm, wn, mfma, stages, swizzle): a spread of the template space used by the parity tests
PARITY_SHAPES = [
    (256, 256, 128, 2, 2, 32, 2, 2),
    (256, 256, 64, 2, 4, 32, 4, 0),
    (128, 128, 128, 2, 2, 32, 2, 1),
    (128, 256, 64, 2, 2, 32, 3, 3),
    (64, 64, 128, 1, 1, 32, 3, 1),
    (128, 128, 128, 2, 2, 16, 2, 1),
    (64, 128, 256, 1, 2, 16, 2, 1),
    (32, 32, 128, 1, 2, 16, 4, 0),
    (256, 256, 128, 2, 4, 16, 2, 2),
]


# (tile tuple) instances run with the LDS-staged epilogue as well
EPILOGUE_VARIANTS = [
    (256, 256, 128, 2, 4, 16, 2, 2),
    (256, 256, 128, 4, 2, 32, 2, 2),
    (256, 256, 128, 4, 2, 16, 2, 2),
    (256, 256, 64, 2, 4, 32, 4, 3),
    (128, 128, 128, 2, 2, 32, 2, 1),
    (64, 64, 128, 4, 2, 16, 3, 1),
    (64, 128, 256, 1, 2, 16, 2, 1),
    (128, 64, 128, 2, 1, 32, 2, 1),
]

# one MFMA k-step per k-tile (64-byte rows with 16x16 MFMAs): the register buffers alternate per tile
SINGLE_STEP_VARIANTS = [
    (256, 256, 64, 2, 4, 16, 5, 3),
    (256, 256, 64, 4, 2, 16, 4, 3),
    (128, 128, 64, 2, 2, 16, 3, 3),
    (64, 64, 64, 1, 2, 16, 2, 3),
]


def variant_descs():
    out = []
    for t in EPILOGUE_VARIANTS + SINGLE_STEP_VARIANTS:
        out.append(D(F16, GEMM, *t, epi=1))
        out.append(D(U8, GEMM, *t, epi=1))
    # two-group schedule (sched 2): 8 waves, one and two k-steps per tile, 2..4 stages, both MFMA shapes, im2col conv
    out.append(D(U8, GEMM, 256, 256, 128, 2, 4, 16, 2, 1, sched=2))
    out.append(D(F16, GEMM, 256, 256, 128, 4, 2, 16, 2, 1, epi=2, sched=2))
    out.append(D(U8, GEMM, 128, 128, 64, 2, 4, 16, 4, 3, epi=1, sched=2))
    out.append(D(F16, GEMM, 128, 256, 64, 2, 4, 32, 3, 2, sched=2))
    out.append(D(F16, CONV, 128, 64, 128, 4, 2, 16, 2, 1, epi=1, sched=2))
    # non-temporal result stores: direct and staged epilogues, both element types
    out.append(D(F16, GEMM, 128, 128, 128, 2, 2, 32, 2, 1, nt=1))
    out.append(D(F16, GEMM, 256, 256, 128, 2, 4, 16, 2, 2, epi=2, nt=1))
    out.append(D(U8, GEMM, 128, 128, 128, 2, 2, 16, 2, 1, epi=1, colsum=1, nt=1))
    # column sums of B supplied by the caller (colsum 1): plain, staged epilogue, two-group schedule
    out.append(D(U8, GEMM, 256, 256, 128, 2, 4, 16, 2, 1, colsum=1))
    out.append(D(U8, GEMM, 64, 128, 256, 1, 2, 16, 2, 1, epi=1, colsum=1))
    out.append(D(U8, GEMM, 128, 128, 128, 2, 2, 32, 2, 1, epi=2, colsum=1))
    out.append(D(U8, GEMM, 256, 256, 128, 2, 4, 16, 2, 1, sched=2, colsum=1))
    out.append(D(F16, GEMM, 64, 64, 64, 1, 2, 16, 2, 3))
    out.append(D(U8, GEMM, 128, 128, 64, 4, 1, 16, 3, 3))
    out.append(D(F16, CONV, 256, 64, 128, 8, 1, 16, 2, 1, epi=1))
    out.append(D(F16, CONV, 256, 64, 128, 8, 1, 16, 2, 1, epi=1, win=1))
    out.append(D(F16, CONV, 128, 64, 128, 2, 2, 32, 3, 1, win=1))
    out.append(D(F16, CONV, 64, 64, 64, 2, 2, 32, 2, 2, epi=1, win=1))
    out.append(D(F16, CONV, 128, 64, 128, 2, 1, 32, 2, 1, epi=1))
    out.append(D(F16, CONV, 128, 64, 64, 4, 1, 16, 3, 3, epi=1))
    out.append(D(F16, CONV, 128, 64, 128, 4, 1, 16, 2, 2, epi=1, win=1))
    return out


def splitk_descs():
    """Split-K instances of the parity suite (GEMM and im2col conv, both element kinds, both epilogues)."""
    return [
        D(F16, GEMM, 64, 64, 128, 2, 2, 16, 3, 1, epi=1, split=1),
        D(F16, GEMM, 128, 64, 64, 2, 2, 32, 3, 2, epi=0, split=1),
        D(U8, GEMM, 64, 64, 128, 2, 2, 16, 3, 1, epi=1, split=1),
        D(U8, GEMM, 64, 128, 128, 1, 2, 32, 2, 1, epi=0, split=1),
        D(F16, CONV, 64, 64, 128, 2, 2, 16, 3, 1, epi=1, split=1),
        D(U8, CONV, 64, 64, 64, 2, 2, 32, 2, 1, epi=1, split=1),
        D(U8, GEMM, 64, 64, 128, 2, 2, 16, 3, 1, epi=1, split=1, colsum=1),
    ]


def parity_descs():
    out = []
    for t in PARITY_SHAPES:
        out.append(D(F16, GEMM, *t))
        out.append(D(U8, GEMM, *t))
    for t in PARITY_SHAPES[:6]:
        bm, bn, bkb, wm, wn, mfma, st, swz = t
        if swz and (wm * wn * (64 // (bkb // 16))) % ((bkb // 16) << (swz - 1)):
            continue
        out.append(D(F16, CONV, *t))
    return out


def int8_conv_descs():
    """uint8 x int8 -> int32 conv2d instances of the parity suite (im2col and window load paths)."""
    return [
        D(U8, CONV, 64, 64, 64, 2, 2, 32, 2, 1),
        D(U8, CONV, 128, 64, 128, 2, 2, 16, 3, 1, epi=1),
        D(U8, CONV, 128, 128, 128, 2, 2, 32, 2, 1, epi=1),
        D(U8, CONV, 64, 32, 128, 2, 1, 16, 4, 0),
        D(U8, CONV, 128, 64, 64, 4, 1, 32, 2, 1, epi=1, win=1),
        D(U8, CONV, 256, 64, 128, 8, 1, 16, 2, 1, win=1),
        D(U8, CONV, 128, 64, 128, 2, 2, 16, 3, 1, epi=1, colsum=1),
        D(U8, CONV, 128, 64, 64, 4, 1, 32, 2, 1, epi=1, win=1, colsum=1),
    ]


def persistent_descs():
    """Instances of the persistent (tile-stream) mode in the parity suite: short and long K streams, both element
    kinds, 2..4 stages, implicit-GEMM conv."""
    return [
        D(F16, GEMM, 128, 128, 64, 2, 4, 32, 2, 1, epi=1, pers=1),
        D(F16, GEMM, 64, 64, 128, 4, 2, 16, 3, 1, epi=1, pers=1),
        D(F16, GEMM, 256, 128, 128, 4, 2, 32, 2, 2, epi=1, pers=1),
        D(F16, GEMM, 256, 128, 128, 4, 2, 16, 2, 2, epi=1, pers=1),
        D(F16, GEMM, 128, 128, 64, 2, 2, 32, 4, 2, epi=1, pers=1),
        D(U8, GEMM, 128, 128, 64, 2, 2, 32, 4, 3, epi=1, pers=1),
        D(U8, GEMM, 64, 128, 256, 1, 2, 16, 2, 1, epi=1, pers=1),
        D(F16, CONV, 128, 64, 128, 2, 1, 32, 2, 1, epi=1, pers=1),
        D(U8, CONV, 128, 64, 128, 2, 2, 16, 3, 1, epi=1, pers=1),
        D(U8, GEMM, 128, 128, 64, 2, 2, 32, 4, 3, epi=1, pers=1, colsum=1),
        D(F16, GEMM, 128, 128, 64, 2, 2, 32, 4, 3, epi=1, pers=1, nt=1),
    ]


def persistent_twin_descs():
    """The one-tile-per-workgroup instances with the same tiles as the persistent GEMM instances (bit-identity checks)."""
    return [D(d.dtype, d.op, *d.as_tuple()[2:10], epi=1) for d in persistent_descs() if d.op == GEMM]


# small general-purpose instances (smoke, error-path and operator tests); the tuned instances of the benchmark
# configurations come from the records under tests/quick_start/rocm/tuned/ (heron_amd.tuned)
BEST = {
    "small": D(U8, GEMM, 64, 64, 128, 1, 1, 32, 3, 1),
    "small_f16": D(F16, GEMM, 64, 64, 128, 1, 1, 32, 3, 1),
}


def all_shipped():
    seen, out = set(), []
    for d in (parity_descs() + variant_descs() + int8_conv_descs() + persistent_descs() + persistent_twin_descs() + splitk_descs()
              + list(BEST.values())):
        if d.as_tuple() not in seen:
            seen.add(d.as_tuple())
            out.append(d)
    return out


def _compile_one(tup):
    d = B.make_desc(*tup)
    try:
        return tup, B.compile_desc(d, 300.0), None
    except Exception as e:  # noqa: BLE001 - reported to the caller
        return tup, None, str(e)


def precompile(descs, jobs=None, verbose=False):
    """Compile descriptors into the cache with ``jobs`` parallel hipcc workers; returns the failures."""
    jobs = jobs or min(8, os.cpu_count() or 1)
    tups = [d.as_tuple() for d in descs]
    failures = []
    with ProcessPoolExecutor(max_workers=jobs) as ex:
        for tup, path, err in ex.map(_compile_one, tups):
            if err:
                failures.append((tup, err))
            if verbose:
                print(("FAIL " + err[:200]) if err else "ok  ", tup, flush=True)
    return failures
