"""Shared pieces of the MFMA operator definitions."""

F16_NAMES = ("float16", "fp16", "half")
I8_NAMES = ("int8", "uint8", "u8s8")


def element_kind(in_dtype):
    """'f16' for fp16 operands, 'u8s8' for the quantized path.

    As in ops/x86/dense.py:10-11 of the reference, the quantized path always takes A as uint8 and
    B as int8 whatever the config's ``in_dtype`` says ("int8" in its JSON files).
    """
    if in_dtype in F16_NAMES:
        return "f16"
    if in_dtype in I8_NAMES:
        return "u8s8"
    raise ValueError("unsupported in_dtype %r for the MFMA templates" % (in_dtype,))


def mfma_info(kind, stage_name, a_name, b_name, gemm_view, operator, extra=None):
    """The ``info`` dictionary an operator hands to ``ctx.set_info``.

    Counterpart of the 'tensorcore' / 'x86_dot' dictionaries (ops/cuda/dense.py:33-43,
    ops/x86/dense.py:21-26): it names the compute stage, how A and B are read, and which hardware
    instruction family the template is built on.
    """
    info = {
        'name': 'mfma',
        'stage_name': stage_name,
        'operator': operator,                      # 'gemm' | 'conv2d_nhwc'
        'kind': kind,                              # 'f16' | 'u8s8'
        'loadA': (a_name, 'k_contiguous'),
        'loadB': (b_name, 'k_contiguous'),        # B is stored (N, K): column-major K x N
        'com': ('mfma', 'float32' if kind == 'f16' else 'int32'),
        'store': ('row_major', 'float16' if kind == 'f16' else 'int32'),
        'gemm_view': gemm_view,                    # dict(batch, M, N, K)
    }
    if extra:
        info.update(extra)
    return info
