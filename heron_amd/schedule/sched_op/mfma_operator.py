"""Schedule operations of the MFMA kernel template, and the CDNA4 constraint set.

In the reference a schedule operation transforms TVM loops and, while the template is being
built, registers the knobs and constraints the transformation implies
(schedule/sched_op/sched_common.py, gpu_common.py, gpu_tensorcore_operator.py).  Here the kernel is
a fixed hand-written HIP template, so an operation only (a) registers knobs/constraints in
building mode and (b) copies the solved values into the ``TemplateSchedule``; replaying
``knob_manager.sched_tups`` with a solved KnobManager therefore yields a concrete template
instance, exactly as ``Task.instantiate`` replays TVM primitives in the reference.

Each constraint cites the reference constraint it replaces.
"""
from ...utils import genKey


class TemplateSchedule:
    """What ``te.create_schedule`` is to the reference: the object the operations fill in."""

    def __init__(self, outs, info):
        self.outs = outs
        self.info = info
        self.params = {}

    def __getitem__(self, key):
        return self.params[key]

    def to_desc(self):
        from ... import backend as B
        p = self.params
        dtype = B.HRN_DT_F16 if self.info['kind'] == 'f16' else B.HRN_DT_U8S8
        op = B.HRN_OP_CONV2D if self.info['operator'] == 'conv2d_nhwc' else B.HRN_OP_GEMM
        return B.make_desc(dtype, op, p['bm'], p['bn'], p['bkb'], p['wm'], p['wn'], p['mfma'], p['stages'],
                           p['swizzle'], p.get('epilogue', 0), p['waves_per_eu'],
                           p.get('conv_window', 0), p.get('persistent', 0), 1 if p.get('split_k', 1) > 1 else 0,
                           p.get('sched', 1), p.get('load_spread', 2), p.get('colsum', 0), p.get('nt_store', 0))

    def to_problem(self):
        from ... import backend as B
        g = self.info['gemm_view']
        if self.info['operator'] == 'conv2d_nhwc':
            c = self.info['conv']
            return B.conv2d_problem(c['N'], c['H'], c['W'], c['CI'], c['CO'], c['KH'], c['KW'],
                                    (c['stride'], c['stride_w']), (c['pad'], c['pad_w']), (c['dil'], c['dil_w']),
                                    self.params['group_m'], self.params.get('split_k', 1))
        return B.gemm_problem(g['batch'], g['M'], g['N'], g['K'], self.params['group_m'], self.params.get('split_k', 1))

    def describe(self):
        return ", ".join("%s=%s" % kv for kv in sorted(self.params.items()))


def roundup(x, m):
    return (x + m - 1) // m * m


class schedOp:
    def __init__(self, name):
        self.name = name

    # --- helpers -----------------------------------------------------------------------
    @staticmethod
    def P(stage, param):
        return genKey("P", stage, param_name=param)

    @staticmethod
    def V(stage, var):
        return genKey("V", stage, var_name=var)

    @staticmethod
    def L(stage, ax):
        return genKey("L", stage, ax)

    def knob(self, ctx, stage, param, candidates, default):
        """A tunable parameter restricted to ``candidates`` (the define_knob + addCandidates idiom of
        gpu_tensorcore_operator.py:285-294)."""
        km = ctx.knob_manager
        key = self.P(stage, param)
        km.define_value(key, min(candidates), max(candidates), default, True)
        if list(candidates) != list(range(min(candidates), max(candidates) + 1)):
            km.addCandidates(key, list(candidates))
        else:
            km.addRawCandidates(key, list(candidates))
        return key

    def var(self, ctx, stage, name, low, up, default=None):
        return ctx.knob_manager.define_value(self.V(stage, name), low, up, low if default is None else default)

    def perform(self, s, stage_name, ctx):
        raise NotImplementedError


class startOp(schedOp):
    """Declares the GEMM view of the stage as loop extents (the role of startOp in sched_common.py:
    axis extents enter the CSP as constants)."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        g, kind = s.info['gemm_view'], s.info['kind']
        es = 2 if kind == 'f16' else 1
        # spatial extents are padded to one 16-row MFMA tile, K (in bytes) to one 64-byte LDS row
        km.axis_ori_lenth[self.L(stage_name, 'i')] = roundup(g['M'], 16)
        km.axis_ori_lenth[self.L(stage_name, 'j')] = roundup(g['N'], 16)
        km.axis_ori_lenth[self.L(stage_name, 'k')] = roundup(g['K'] * es, 64)
        km.axis_ori_lenth[self.L(stage_name, 'b')] = g['batch']
        ctx.addSchedDesc("\n## Stage %s: %s %s, GEMM view batch=%d M=%d N=%d K=%d\n" % (
            stage_name, s.info['operator'], kind, g['batch'], g['M'], g['N'], g['K']))


class mfmaShapeOp(schedOp):
    """MFMA instruction shape: 32x32x(16 f16 | 32 i8) or 16x16x(32 f16 | 64 i8); both consume 1024
    operand bytes per wave.  Replaces the wmma m/n/k candidates [8,16,32] with m*n*k = 4096
    (gpu_tensorcore_operator.py:285-294)."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        mfma = self.knob(ctx, stage_name, 'mfma', [16, 32], 32)
        ksb = self.var(ctx, stage_name, 'mfma_k_bytes', 32, 64, 32)
        km.addProd([mfma, ksb], 1024)
        m2 = self.var(ctx, stage_name, 'mfma_area', 256, 1024, 1024)
        km.addProd([mfma, mfma], m2)
        apt = self.var(ctx, stage_name, 'acc_regs_per_tile', 4, 16, 16)
        km.addProd([64, apt], m2)                     # one accumulator register per 64 outputs
        s.params['mfma'] = km.get_val(mfma)
        ctx.addSchedDesc("mfma = %s  # %s\n" % (km.get_val(mfma), mfma))


class tileWaveOp(schedOp):
    """Wave grid and per-wave MFMA tiling: lanes per wave are fixed at 64 (replaces
    addEQ(threadIdx.x, 32), gpu_common.py:36-37) and waves = wm*wn <= max_threads/64 (replaces
    threads <= 1024, cuda_context.py:25-32)."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        max_waves = ctx.getLimit('max_threads_per_wg') // ctx.getLimit('wave_size')
        wm = self.knob(ctx, stage_name, 'wave_m', [1, 2, 4, 8], 2)
        wn = self.knob(ctx, stage_name, 'wave_n', [1, 2, 4, 8], 2)
        waves = self.var(ctx, stage_name, 'waves', 1, max_waves, 4)
        km.addProd([wm, wn], waves)
        tm = self.knob(ctx, stage_name, 'tile_m', list(range(1, 17)), 2)
        tn = self.knob(ctx, stage_name, 'tile_n', list(range(1, 17)), 2)
        mfma = self.P(stage_name, 'mfma')
        wtm = self.var(ctx, stage_name, 'wave_tile_m', 16, 512, 64)
        wtn = self.var(ctx, stage_name, 'wave_tile_n', 16, 512, 64)
        km.addProd([tm, mfma], wtm)
        km.addProd([tn, mfma], wtn)
        for k, key in (('wm', wm), ('wn', wn), ('tm', tm), ('tn', tn)):
            s.params[k] = km.get_val(key)
        ctx.addSchedDesc("wave grid = %s x %s, mfma tiles per wave = %s x %s\n" % tuple(
            km.get_val(k) for k in (wm, wn, tm, tn)))


class tileBlockOp(schedOp):
    """Workgroup tile: bm = wm * wave_tile_m and grid_m = ceil(M / bm) (and the same for N).  The reference's split
    chain is exact (extent = outer * inner, knobManager.py:83-107) because TVM splits must divide; the kernel
    guards ragged edge tiles itself, so the chain here is the covering form
    grid * b = extent + waste, 0 <= waste < b, which keeps shapes with awkward factors (149 * 149 pixels) tunable."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        for ax, w, wt, b, g in (('i', 'wave_m', 'wave_tile_m', 'block_m', 'grid_m'),
                                ('j', 'wave_n', 'wave_tile_n', 'block_n', 'grid_n')):
            extent = km.axis_ori_lenth[self.L(stage_name, ax)]
            bkey = self.var(ctx, stage_name, b, 16, min(512, extent), 16)
            gkey = self.var(ctx, stage_name, g, 1, extent // 16, extent // 16)
            km.addProd([self.P(stage_name, w), self.V(stage_name, wt)], bkey)
            cover = self.var(ctx, stage_name, g + '_cover', extent, extent + 511, extent)
            waste = self.var(ctx, stage_name, g + '_waste', 0, 511, 0)
            km.addProd([gkey, bkey], cover)
            km.addSUM(cover, [extent, waste])
            km.addLT(waste, bkey)
            s.params['bm' if ax == 'i' else 'bn'] = km.get_val(bkey)
        ctx.addSchedDesc("block tile = %s x %s\n" % (s.params['bm'], s.params['bn']))


class tileKOp(schedOp):
    """K tiling: bkb bytes of K per LDS row = 1, 2, 4 or 8 MFMA k-steps per tile, and k_tiles =
    ceil(K_bytes / bkb) (the split constraint of the reduce axis, sched_common.py generalTileOp, in covering form:
    the part of the last tile past the end of K is fetched as zeros)."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        kbytes = km.axis_ori_lenth[self.L(stage_name, 'k')]
        bkb = self.knob(ctx, stage_name, 'block_k_bytes', [64, 128, 256], 128)
        ks = self.var(ctx, stage_name, 'k_steps', 1, 8, 4)
        km.addCandidates(ks, [1, 2, 4, 8])
        km.addProd([ks, self.V(stage_name, 'mfma_k_bytes')], bkb)
        kt = self.var(ctx, stage_name, 'k_tiles', 1, kbytes // 64, kbytes // 64)
        kcover = self.var(ctx, stage_name, 'k_cover', kbytes, kbytes + 255, kbytes)
        kwaste = self.var(ctx, stage_name, 'k_waste', 0, 255, 0)
        km.addProd([kt, bkb], kcover)
        km.addSUM(kcover, [kbytes, kwaste])
        km.addLT(kwaste, bkb)
        s.params['bkb'] = km.get_val(bkb)
        ctx.addSchedDesc("k tile = %s bytes\n" % s.params['bkb'])


class convWindowOp(schedOp):
    """conv2d only: 1 keeps the window of input pixels the tile's outputs can reach (bm + 2*pad*(W+1) pixels, all
    channels) in LDS and reads every filter tap from it; 0 fetches an im2col tile of A per tap.  Window mode needs
    stride 1, dilation 1, 'same' padding, at most 32 taps and whole k-tiles per pixel (CI*elem_bytes = q * bkb).  It plays the
    role of the reference's compute_at choice for the padded-input stage (GPUfinishOp position knobs,
    gpu_common.py:154-223): where the shared copy of the input lives relative to the reduction loops."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        ok = False
        pitch = 16
        halo = 0
        if s.info['operator'] == 'conv2d_nhwc':
            c = s.info['conv']
            ok = (c['stride'] == 1 and c['dil'] == 1 and c['stride_w'] == 1 and c['dil_w'] == 1 and
                  c['HO'] == c['H'] and c['WO'] == c['W'] and c['KH'] * c['KW'] <= 32)
            pitch = c['CI'] * (2 if s.info['kind'] == 'f16' else 1)
            halo = 2 * (c['pad'] * c['W'] + c['pad_w'])
        win = self.knob(ctx, stage_name, 'conv_window', [0, 1] if ok else [0], 0)
        staged = self.var(ctx, stage_name, 'a_rows_staged', 0, 512, 16)       # rows of A that go through the stages
        off = self.var(ctx, stage_name, 'conv_window_off', 0, 1, 1)
        km.addSUM(1, [win, off])
        km.addProd([off, self.V(stage_name, 'block_m')], staged)
        # window bytes (0 when off) and whole k-tiles per pixel
        rows = self.var(ctx, stage_name, 'window_rows', 16, 512 + halo, 16 + halo)
        km.addSUM(rows, [self.V(stage_name, 'block_m'), halo])
        wb = self.var(ctx, stage_name, 'window_bytes_full', 256, (512 + halo) * pitch, 256)
        km.addProd([pitch, rows], wb)
        used = self.var(ctx, stage_name, 'window_bytes', 0, ctx.getLimit('lds_bytes_per_wg'), 0)
        km.addProd([win, wb], used)
        pw = self.var(ctx, stage_name, 'window_pitch_used', 0, pitch, 0)
        km.addProd([win, pitch], pw)
        q = self.var(ctx, stage_name, 'window_k_tiles_per_pixel', 0, max(1, pitch // 64), 0)
        km.addProd([q, self.P(stage_name, 'block_k_bytes')], pw)
        s.params['conv_window'] = km.get_val(win)
        ctx.addSchedDesc("conv window mode = %s\n" % s.params['conv_window'])


class loadVectorOp(schedOp):
    """Global->LDS transfer: every lane moves one 128-bit chunk per load and one wave instruction fills
    1 KiB of LDS, so a tile must split into whole wave loads: bm = loads_a * (64/chunks_per_row) * waves.
    Replaces the vectorize candidates [1,2,4,8] halfs and their stride filter
    (gpu_tensorcore_operator.py:15-21): the width is fixed at 16 bytes, the divisibility is what remains."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        bkb = self.P(stage_name, 'block_k_bytes')
        cpr = self.var(ctx, stage_name, 'chunks_per_row', 4, 16, 8)
        km.addProd([16, cpr], bkb)
        rpi = self.var(ctx, stage_name, 'rows_per_load', 4, 16, 8)
        km.addProd([rpi, cpr], 64)
        rpr = self.var(ctx, stage_name, 'rows_per_round', 4, 256, 32)
        km.addProd([rpi, self.V(stage_name, 'waves')], rpr)
        la = self.var(ctx, stage_name, 'loads_a', 1, 32, 1)
        lb = self.var(ctx, stage_name, 'loads_b', 1, 32, 1)
        km.addProd([la, rpr], self.V(stage_name, 'block_m'))
        km.addProd([lb, rpr], self.V(stage_name, 'block_n'))
        lpt = self.var(ctx, stage_name, 'loads_per_tile', 2, 64, 2)
        km.addSUM(lpt, [la, lb])
        ctx.addSchedDesc("global->LDS: 16-byte chunks, direct to LDS\n")


class ldsStageOp(schedOp):
    """LDS staging: stages * (bm + bn) * bkb <= LDS bytes per workgroup (replaces shared_mem_size <=
    max_shared_memory_per_block/2 elements, cuda_context.py:45-63), and the loads in flight
    (stages-1) * loads_per_tile must fit the 6-bit vmcnt counter."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        lds_limit = ctx.getLimit('lds_bytes_per_wg')
        stages = self.knob(ctx, stage_name, 'lds_stages', [2, 3, 4, 5], 2)
        bmn = self.var(ctx, stage_name, 'block_m_plus_n', 16, 1024, 32)
        km.addSUM(bmn, [self.V(stage_name, 'a_rows_staged'), self.V(stage_name, 'block_n')])
        sb = self.var(ctx, stage_name, 'stage_bytes', 1024, lds_limit // 2, 2048)
        km.addProd([bmn, self.P(stage_name, 'block_k_bytes')], sb)
        lds = self.var(ctx, stage_name, 'lds_bytes', 2048, lds_limit, 4096)
        km.addProd([stages, sb], lds)
        # the conv window (dynamic LDS, rounded up to whole 1 KiB wave loads) shares the budget
        with_win = self.var(ctx, stage_name, 'lds_bytes_with_window', 2048, lds_limit - 1024, 4096)
        km.addSUM(with_win, [lds, self.V(stage_name, 'window_bytes')])
        if lds not in km.mems:
            km.mems.append(lds)
        ahead = self.var(ctx, stage_name, 'stages_ahead', 1, 4, 1)
        km.addSUM(stages, [ahead, 1])
        inflight = self.var(ctx, stage_name, 'loads_in_flight', 1, ctx.getLimit('max_loads_in_flight'), 1)
        km.addProd([ahead, self.V(stage_name, 'loads_per_tile')], inflight)
        s.params['stages'] = km.get_val(stages)
        ctx.addSchedDesc("LDS stages = %s\n" % s.params['stages'])


class ldsSwizzleOp(schedOp):
    """XOR swizzle of the 16-byte chunks of an LDS row with (row >> (swizzle-1)); its period
    chunks_per_row << (swizzle-1) must not exceed the MFMA tile edge.  Replaces the storage_align
    offsets [0,8,16,24,32,48] (gpu_common.py:133-152): padding is impossible with direct-to-LDS
    loads (one instruction writes 1 KiB contiguously), swizzling does the same job."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        swz = self.knob(ctx, stage_name, 'lds_swizzle', [0, 1, 2, 3], 1)
        cpr = self.V(stage_name, 'chunks_per_row')
        p2 = self.var(ctx, stage_name, 'swizzle_period2', 8, 32, 16)
        p4 = self.var(ctx, stage_name, 'swizzle_period4', 16, 64, 32)
        km.addProd([2, cpr], p2)
        km.addProd([4, cpr], p4)
        period = self.var(ctx, stage_name, 'swizzle_period', 1, 32, 8)
        km.addSelect([1, cpr, p2, p4], swz, period)
        km.addLE(period, self.P(stage_name, 'mfma'))
        if s.info['operator'] == 'conv2d_nhwc':
            # the lane's chunk column must be the same for every load of a tile
            q = self.var(ctx, stage_name, 'rounds_per_period', 1, 256, 1)
            km.addProd([q, period], self.V(stage_name, 'rows_per_round'))
        s.params['swizzle'] = km.get_val(swz)
        ctx.addSchedDesc("LDS swizzle = %s\n" % s.params['swizzle'])


class registerBudgetOp(schedOp):
    """Register file: accumulators tm*tn*(mfma^2/64) <= 256 per lane, plus operand fragments and a fixed
    allowance for addresses; times the waves each SIMD hosts (waves/4, at least 1) it must fit the
    512-entry unified VGPR+AGPR file.  The fragment term 6*(tm+tn) and the allowance are fitted to what
    hipcc allocates for compiled instances (it keeps less than two full fragment sets live): 256x256
    tiles on 8 waves take 200 registers with 32x32 MFMAs (tm+tn = 6) and 226-247 with 16x16 MFMAs
    (tm+tn = 12), both of which must stay in the space.  No counterpart in the reference (NVCC
    allocates registers behind TVM's back)."""

    OVERHEAD = 32
    FRAG_REGS = 6

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        regs_total = ctx.getLimit('regs_per_simd_lane')
        simds = ctx.getLimit('simd_per_cu')
        tm, tn = self.P(stage_name, 'tile_m'), self.P(stage_name, 'tile_n')
        tmn = self.var(ctx, stage_name, 'tiles_per_wave', 1, 128, 4)
        km.addProd([tm, tn], tmn)
        acc = self.var(ctx, stage_name, 'acc_regs', 4, regs_total // 2, 64)
        km.addProd([tmn, self.V(stage_name, 'acc_regs_per_tile')], acc)
        tsum = self.var(ctx, stage_name, 'tile_m_plus_n', 2, 32, 4)
        km.addSUM(tsum, [tm, tn])
        frag = self.var(ctx, stage_name, 'frag_regs', 6, 256, 36)
        km.addProd([self.FRAG_REGS, tsum], frag)
        regs = self.var(ctx, stage_name, 'regs_per_lane', 1, regs_total, 128)
        km.addSUM(regs, [acc, frag, self.OVERHEAD])
        # waves of one workgroup that share a SIMD
        waves = self.V(stage_name, 'waves')
        wps = self.var(ctx, stage_name, 'waves_per_simd', 1, 4, 1)
        max_waves = ctx.getLimit('max_threads_per_wg') // ctx.getLimit('wave_size')
        cands = [w for w in (1, 2, 4, 8, 16) if w <= max_waves]
        km.addCandidates(waves, cands)
        from ..constraints.primitives import EQ
        if km.is_building:
            for idx, w in enumerate(cands):
                km.solver.primitives.append(EQ([wps, max(1, w // simds)], cond="O#" + waves + '_cand%d' % idx))
        budget = self.var(ctx, stage_name, 'regs_per_simd', 1, regs_total, 128)
        km.addProd([regs, wps], budget)
        hint = self.knob(ctx, stage_name, 'waves_per_eu', [0, 1, 2], 0)
        hinted = self.var(ctx, stage_name, 'regs_hinted', 0, regs_total, 0)
        km.addProd([hint, regs], hinted)
        s.params['waves_per_eu'] = km.get_val(hint)
        ctx.addSchedDesc("occupancy hint = %s\n" % s.params['waves_per_eu'])


class splitKOp(schedOp):
    """Split-K: the reduction is cut into ``split_k`` slices that run as separate workgroups and a second pass adds
    their partial sums (for small M*N with long K, where the output tiles alone cannot fill the CUs).  A slice holds
    at least one k-tile; splitting is only offered while the output tiles number at most one per CU, and it
    excludes the input window and (in persistentOp) the persistent launch.  The kernel then writes 4-byte partial sums
    whatever the element type.  The reference never splits the reduce axis over blocks (ops/cuda/dense.py:18-26 binds
    only spatial axes to blockIdx); its counterpart is the rfactor-free reduce split of generalTileOp."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        g = s.info['gemm_view']
        cus = ctx.getLimit('cu_count')
        cands = [1, 2, 4, 8, 16]
        sk = self.knob(ctx, stage_name, 'split_k', cands, 1)
        km.addCandidates(sk, cands)
        on = self.var(ctx, stage_name, 'split_k_on', 0, 1, 0)
        km.addSUM(1, [on, sk.replace("P#", "O#") + '_cand0'])
        km.addLE(sk, self.V(stage_name, 'k_tiles'))
        tiles = self.var(ctx, stage_name, 'output_tiles', 1, 1 << 24, 1)
        km.addProd([self.V(stage_name, 'grid_m'), self.V(stage_name, 'grid_n')], tiles)
        gated = self.var(ctx, stage_name, 'split_k_output_tiles', 0, max(1, cus // max(1, g['batch'])), 0)
        km.addProd([on, tiles], gated)
        sw = self.var(ctx, stage_name, 'split_k_plus_window', 0, 1, 0)
        km.addSUM(sw, [on, self.P(stage_name, 'conv_window')])
        # bytes of an output element as the kernel stores it
        oes = self.var(ctx, stage_name, 'out_elem_bytes', 2, 4, 4)
        if s.info['kind'] == 'f16':
            extra = self.var(ctx, stage_name, 'out_elem_bytes_extra', 0, 2, 0)
            km.addProd([2, on], extra)
            km.addSUM(oes, [2, extra])
        else:
            km.addEQ(oes, 4)
        s.params['split_k'] = km.get_val(sk)
        ctx.addSchedDesc("split_k = %s\n" % s.params['split_k'])


class epilogueOp(schedOp):
    """Result write-back: 0 stores 8/16-byte pieces straight from the accumulator registers; 1 parks one MFMA row-tile
    per wave in a padded LDS strip as wide as the wave tile and streams it out 16 bytes per lane (whole row segments
    per store); 2 does the same through strips of half that width, filled twice per row-tile (half the LDS, which is
    what lets a 256x256 int32 tile keep its stages live in persistent mode).  The strips must fit the LDS budget and
    split into whole wave stores.  Replaces the store stage of the reference's TensorCore template (tensorcoreStoreOp
    through shared memory, gpu_tensorcore_operator.py), where it is not a choice."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        lds_limit = ctx.getLimit('lds_bytes_per_wg')
        epi = self.knob(ctx, stage_name, 'epilogue', [0, 1, 2], 1)
        km.addCandidates(epi, [0, 1, 2])
        oh = epi.replace("P#", "O#")
        on = self.var(ctx, stage_name, 'epilogue_staged', 0, 1, 1)
        km.addSUM(1, [on, oh + '_cand0'])
        # strips per row-tile (1 or 2) and their width in outputs: strips * strip_width = wave_tile_n, whole MFMA tiles each
        nstr = self.var(ctx, stage_name, 'epi_strips', 1, 2, 1)
        km.addSUM(nstr, [1, oh + '_cand2'])
        sw = self.var(ctx, stage_name, 'epi_strip_width', 8, 512, 64)
        km.addProd([nstr, sw], self.V(stage_name, 'wave_tile_n'))
        tns = self.var(ctx, stage_name, 'epi_tiles_per_strip', 1, 16, 1)
        km.addProd([nstr, tns], self.P(stage_name, 'tile_n'))
        row = self.var(ctx, stage_name, 'epi_row_bytes', 32, 2048, 64)
        km.addProd([self.V(stage_name, 'out_elem_bytes'), sw], row)
        pitch = self.var(ctx, stage_name, 'epi_pitch', 48, 2064, 80)
        km.addSUM(pitch, [row, 16])
        lanes = self.var(ctx, stage_name, 'epi_rows_all', 16, 512, 32)
        km.addProd([self.V(stage_name, 'waves'), self.P(stage_name, 'mfma')], lanes)
        strips = self.var(ctx, stage_name, 'epi_strip_bytes', 768, lds_limit * 8, 768)
        km.addProd([lanes, pitch], strips)
        base = 0
        if s.info['kind'] != 'f16':
            # column sums of B: one row of block_n sums per wave row, rounded up to 1 KiB
            base = self.var(ctx, stage_name, 'epi_base', 1024, 16384, 1024)
            kb = self.var(ctx, stage_name, 'epi_base_kib', 1, 16, 1)
            km.addProd([1024, kb], base)
            bn4 = self.var(ctx, stage_name, 'block_n_bytes4', 64, 2048, 64)
            km.addProd([4, self.V(stage_name, 'block_n')], bn4)
            sums = self.var(ctx, stage_name, 'column_sum_bytes', 64, 16384, 64)
            km.addProd([self.P(stage_name, 'wave_m'), bn4], sums)
            km.addLE(sums, base)
            slack = self.var(ctx, stage_name, 'column_sum_bytes_plus_1023', 1087, 17407, 1087)
            km.addSUM(slack, [sums, 1023])
            km.addLE(base, slack)                               # base is the smallest whole KiB that holds the sums
        need = self.var(ctx, stage_name, 'epi_lds_needed', 768, lds_limit * 8 + 16384, 768)
        km.addSUM(need, [strips, base])
        used = self.var(ctx, stage_name, 'epi_lds_bytes', 0, lds_limit, 0)
        km.addProd([on, need], used)                        # 0 when the register epilogue is chosen
        # window mode: the region takes the place of the window (dynamic LDS) next to the filter stages
        ew = self.var(ctx, stage_name, 'epi_lds_bytes_in_window', 0, lds_limit, 0)
        km.addProd([self.P(stage_name, 'conv_window'), used], ew)
        tot = self.var(ctx, stage_name, 'lds_bytes_with_epi_in_window', 2048, lds_limit, 4096)
        km.addSUM(tot, [self.V(stage_name, 'lds_bytes'), ew])
        # a strip must split into whole 1 KiB wave stores: mfma * row_bytes = 1024 * q
        area = self.var(ctx, stage_name, 'epi_strip_area', 512, 65536, 1024)
        km.addProd([self.P(stage_name, 'mfma'), row], area)
        area_e = self.var(ctx, stage_name, 'epi_strip_area_used', 0, 65536, 0)
        km.addProd([on, area], area_e)
        q = self.var(ctx, stage_name, 'epi_wave_stores', 0, 64, 0)
        km.addProd([1024, q], area_e)
        s.params['epilogue'] = km.get_val(epi)
        ctx.addSchedDesc("epilogue = %s\n" % s.params['epilogue'])


class persistentOp(schedOp):
    """Launch shape: 0 = one output tile per workgroup, 1 = as many workgroups as the device holds at once, each
    walking several output tiles with the k-tiles of all of them in one stream through the LDS stages, so the next
    tile's fetches overlap the current tile's stores.  Needs the LDS-staged epilogue in its own LDS region (the
    stages stay live), no input window, no split-K, an even number of k-steps per tile, and the epilogue's store instructions must fit the
    vector-memory counter together with the fetches issued behind them.  No counterpart in the reference (TVM
    launches one thread block per output tile)."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        lds_limit = ctx.getLimit('lds_bytes_per_wg')
        pers = self.knob(ctx, stage_name, 'persistent', [0, 1], 0)
        km.addLE(pers, self.V(stage_name, 'epilogue_staged'))
        pw = self.var(ctx, stage_name, 'persistent_plus_window', 0, 1, 0)
        km.addSUM(pw, [pers, self.P(stage_name, 'conv_window')])
        ps1 = self.var(ctx, stage_name, 'persistent_plus_split', 0, 1, 0)
        km.addSUM(ps1, [pers, self.V(stage_name, 'split_k_on')])
        # the register buffers must be back in phase at the end of every k-tile: an even number of k-steps
        po = self.var(ctx, stage_name, 'persistent_plus_single_step', 0, 1, 0)
        km.addSUM(po, [pers, "O#" + self.V(stage_name, 'k_steps') + '_cand0'])
        pe = self.var(ctx, stage_name, 'persistent_epi_bytes', 0, lds_limit, 0)
        km.addProd([pers, self.V(stage_name, 'epi_lds_needed')], pe)
        tot = self.var(ctx, stage_name, 'lds_bytes_persistent', 2048, lds_limit, 4096)
        km.addSUM(tot, [self.V(stage_name, 'lds_bytes'), pe])
        a2 = self.var(ctx, stage_name, 'stages_ahead_minus_1', 0, 3, 0)
        km.addSUM(self.V(stage_name, 'stages_ahead'), [a2, 1])
        fl = self.var(ctx, stage_name, 'fetches_behind_stores', 0, 63, 0)
        km.addProd([a2, self.V(stage_name, 'loads_per_tile')], fl)
        st = self.var(ctx, stage_name, 'stores_per_tile', 0, 512, 0)
        km.addProd([self.P(stage_name, 'tile_m'), self.V(stage_name, 'epi_strips'), self.V(stage_name, 'epi_wave_stores')], st)
        ps = self.var(ctx, stage_name, 'persistent_stores', 0, 63, 0)
        km.addProd([pers, st], ps)
        vm = self.var(ctx, stage_name, 'persistent_vmem_in_flight', 0, 63, 0)
        km.addSUM(vm, [fl, ps])
        s.params['persistent'] = km.get_val(pers)
        ctx.addSchedDesc("persistent = %s\n" % s.params['persistent'])


class rasterOp(schedOp):
    """Launch-time tile raster: workgroups are spread over the 8 XCDs and walk the tile grid in column
    groups of ``group_m`` row-tiles so that one XCD's L2 holds a compact block of A and B.  Also the issue-order
    style of a k-step: 1 pins the template's own interleaving of fragment reads, tile loads and MFMAs with scheduling
    fences, 0 leaves it to the compiler under group hints (what TVM's generated code leaves to NVCC); and how far the
    wave loads of the next k-tile are spread over the MFMA rows of the step that issues them (0 = all right behind
    the barrier ... 3 = all rows but the last two): the workgroups of an XCD reach that barrier together, so spreading
    smooths the demand on the L2."""

    def perform(self, s, stage_name, ctx):
        km = ctx.knob_manager
        gm = self.knob(ctx, stage_name, 'raster_group_m', [1, 2, 4, 8, 16, 32], 8)
        sc = self.knob(ctx, stage_name, 'issue_order', [0, 1], 1)
        sp = self.knob(ctx, stage_name, 'load_spread', [0, 1, 2, 3], 2)
        # uint8 x int8: where the column sums of B come from (0 = added up in the kernel's k-loop, 1 = supplied with
        # the weights, hrn_colsum_s8); fp16 has no such term
        cs = self.knob(ctx, stage_name, 'column_sums', [0, 1] if s.info['kind'] == 'u8s8' else [0], 0)
        s.params['group_m'] = km.get_val(gm)
        s.params['sched'] = km.get_val(sc)
        s.params['load_spread'] = km.get_val(sp)
        s.params['colsum'] = km.get_val(cs)
        # cache policy of the result stores: 1 = non-temporal (C does not displace the operand slabs in L2); split-K
        # partial sums are read back at once and keep the default policy in either case
        nt = self.knob(ctx, stage_name, 'streaming_store', [0, 1], 0)
        s.params['nt_store'] = km.get_val(nt)
        ctx.addSchedDesc("raster group_m = %s, issue order = %s\n" % (s.params['group_m'], s.params['sched']))


class finishOp(schedOp):
    def perform(self, s, stage_name, ctx):
        ctx.addSchedDesc("# template instance: %s\n" % s.describe())


all_op_methods = {
    'start': startOp,
    'mfmaShape': mfmaShapeOp,
    'tileWave': tileWaveOp,
    'tileBlock': tileBlockOp,
    'tileK': tileKOp,
    'convWindow': convWindowOp,
    'loadVector': loadVectorOp,
    'ldsStage': ldsStageOp,
    'ldsSwizzle': ldsSwizzleOp,
    'registerBudget': registerBudgetOp,
    'splitK': splitKOp,
    'epilogue': epilogueOp,
    'persistent': persistentOp,
    'raster': rasterOp,
    'finish': finishOp,
}

RULE_ORDER = ['start', 'mfmaShape', 'tileWave', 'tileBlock', 'tileK', 'convWindow', 'loadVector', 'ldsStage', 'ldsSwizzle',
              'registerBudget', 'splitK', 'epilogue', 'persistent', 'raster', 'finish']


def sched_via_rule(ctx, s):
    """Apply the rule sequence to the compute stage (the counterpart of
    gpu_tensorcore_operator.py:362-414; one stage, since loads, MFMA and store are fused in the template)."""
    stage_name = ctx.tensorize_info['stage_name']
    for name in RULE_ORDER:
        ctx.addSched(name, stage_name, s)
