"""CDNA4 (gfx950) schedule context: the hardware limits the constraint set is built from.

Plays the role of TENSORCOREContext (schedule/context/cuda_context.py:8-107): where that one
reads ``build_kwargs['check_gpu']`` for the shared-memory and thread limits, this one reads the
same dictionary as filled from ``hrn_device_info`` (LDS bytes per workgroup, threads per
workgroup, wave size, registers per SIMD lane, SIMDs per CU, CU count).
"""
from .context import Context

# limits of MI355X / gfx950, used when no device was queried (e.g. constraint tests on a CPU host)
GFX950_LIMITS = {
    'lds_bytes_per_wg': 163840,
    'max_threads_per_wg': 1024,
    'wave_size': 64,
    'regs_per_simd_lane': 512,     # unified VGPR + AGPR file
    'simd_per_cu': 4,
    'cu_count': 256,
    'max_loads_in_flight': 63,     # vmcnt is a 6-bit counter
}


class CDNA4Context(Context):
    def __init__(self, knob_manager, build_kwargs, target_name):
        Context.__init__(self, knob_manager, build_kwargs, target_name)
        self.codegen_type = 'GPU_MFMA'
        self.is_mfma = True
        self.stage_orgnize = None
        self.limits = dict(GFX950_LIMITS)
        if build_kwargs and 'check_gpu' in build_kwargs:
            for k, v in build_kwargs['check_gpu'].items():
                if k in self.limits and isinstance(v, int) and v > 0:
                    self.limits[k] = v

    def set_info(self, info):
        assert info['name'] == 'mfma'
        self.tensorize_info = info
        self.stage_orgnize = "MFMA_format"

    def getLimit(self, name):
        return self.limits[name]
