"""What the cost model sees of an MFMA template instance.

The reference feeds its boosted trees the raw value of every solver variable (tuner/tuner.py:322-323,
model/xgboost_cost_model.py:100).  For this template that is ~150 numbers, most of them one-hot selectors and
intermediate products, and a search of a few hundred trials cannot sort them out.  ``featurize`` reduces a solved
point to the 16 knobs, a dozen derived quantities (tile, waves, LDS, registers, output tiles per CU, operand reuse)
and the logarithm of an analytic time estimate; ``analytic_seconds`` is that estimate: rounds of workgroups per CU
times the longer of a tile's MFMA time and its L2 -> LDS fetch time, plus fixed per-workgroup and per-launch
costs.  Before anything has been measured the estimate itself ranks the candidates.
"""
import math

KNOBS = ('mfma', 'wave_m', 'wave_n', 'tile_m', 'tile_n', 'block_k_bytes', 'conv_window', 'persistent', 'lds_stages',
         'lds_swizzle', 'waves_per_eu', 'epilogue', 'split_k', 'raster_group_m', 'issue_order', 'load_spread', 'column_sums',
         'streaming_store')
DERIVED = ('block_m', 'block_n', 'waves', 'k_steps', 'k_tiles', 'grid_m', 'grid_n', 'lds_bytes', 'window_bytes',
           'regs_per_lane', 'loads_per_tile')

CUS = 256
PEAK = {'f16': 2.5e15, 'int8': 5.0e15}
MFMA_EFF = 0.62             # of the published peak: what a dense MFMA loop sustains on real data
FETCH_PER_CU = 60e9         # bytes/s one CU draws from the L2s when all CUs do
HBM = 4.0e12
WG_FIXED = 2.5e-6           # prologue + epilogue of a workgroup that cannot hide behind a co-resident one
LAUNCH = 3.0e-6
BARRIER = 0.12e-6           # one workgroup barrier with the waits around it


def _get(values, stage, name, knob):
    key = ("P#ST:%s,AX:None,PA:%s" if knob else "V#ST:%s,AX:None,VA:%s") % (stage, name)
    return values.get(key, 0)


def lds_conflict_ways(bkb, swizzle):
    """Ways of bank conflict of one fragment read: 16 lanes (rows r..r+15, one 16-byte chunk each) are served per LDS
    cycle by 64 banks of 4 bytes, i.e. 16 slots of 16 bytes; the rows hit 16/cpr distinct slots without swizzle and
    min(16, cpr << (swizzle-1)) with it (cpr = 16-byte chunks per row)."""
    cpr = max(1, bkb // 16)
    distinct = max(1, 16 // cpr) if swizzle == 0 else min(16, cpr << (swizzle - 1))
    return 16 // distinct


def analytic_seconds(info, v):
    """Estimated seconds of one launch; ``v`` maps knob / derived names to values."""
    g = info['gemm_view']
    es = 2 if info['kind'] == 'f16' else 1
    bm, bn, bkb = max(1, v['block_m']), max(1, v['block_n']), max(64, v['block_k_bytes'])
    split = max(1, v['split_k'])
    tiles = max(1, v['grid_m']) * max(1, v['grid_n']) * g['batch'] * split
    kbytes = g['K'] * es / split
    lds = v['lds_bytes'] + v['window_bytes'] + (0 if not v['persistent'] else 16384)
    waves = max(1, v['waves'])
    wm, wn = max(1, v['wave_m']), max(1, v['wave_n'])
    per_cu = max(1, min(163840 // max(lds, 1), 512 // max(1, v['regs_per_lane'] * max(1, waves // 4)), 32 // waves, 8))
    on_busiest_cu = math.ceil(tiles / CUS)                      # workgroups the busiest CU runs, side by side or in turn
    # MFMA time of one tile: fewer than two waves per SIMD leave the matrix pipe idle while a wave waits
    occupancy = min(1.0, 0.55 + 0.225 * min(2.0, waves * min(per_cu, on_busiest_cu) / 4.0))
    shape = 1.0 if v['mfma'] == 16 else 0.93                    # 16x16 MFMAs draw less power: higher sustained clock
    t_mfma = 2.0 * bm * bn * (kbytes / es) / (PEAK['f16' if info['kind'] == 'f16' else 'int8'] / CUS * MFMA_EFF * occupancy * shape)
    # global -> LDS: half-line rows (64 bytes) fetch every cache line twice
    a_rows = 0 if v['conv_window'] else bm
    t_fetch = (a_rows + bn) * kbytes / FETCH_PER_CU * (1.25 if bkb == 64 else 1.0)
    # LDS -> registers: every wave reads its rows of A and of B; 256 bytes per clock when conflict-free
    frag_bytes = (wn * bm + wm * bn) * kbytes
    t_lds = frag_bytes * lds_conflict_ways(bkb, v['lds_swizzle']) / (256 * 2.1e9)
    parts = sorted((t_mfma, t_fetch, t_lds))
    k_tiles = max(1, math.ceil(kbytes / bkb))
    sync = k_tiles * BARRIER * (1.0 + waves / 16.0) * (0.6 if v['lds_stages'] > 2 else 1.0)
    # Throughput work (matrix pipe, fetch path, LDS: shared by the workgroups of a CU) adds up over all the CU's
    # workgroups; waiting (barriers, start-up and drain of a workgroup) is paid once per round of co-resident ones.
    t_busy = parts[2] + 0.35 * parts[1] + 0.1 * parts[0]                                # the three overlap only partly
    t_wait = sync + WG_FIXED
    rounds = math.ceil(on_busiest_cu / per_cu)
    out_bytes = 2 if info['kind'] == 'f16' else 4
    moved = g['batch'] * (g['M'] * g['K'] * es + g['N'] * g['K'] * es + g['M'] * g['N'] * out_bytes)
    if split > 1:
        moved += 2 * split * g['batch'] * g['M'] * g['N'] * 4      # partial sums written and read back
    return max(on_busiest_cu * t_busy + rounds * t_wait, moved / HBM) + LAUNCH * (2 if split > 1 else 1)


def featurize(info, values):
    """Feature vector of a solved point (``values``: solver variable name -> value)."""
    stage = info['stage_name']
    v = {k: _get(values, stage, k, True) for k in KNOBS}
    v.update({k: _get(values, stage, k, False) for k in DERIVED})
    g = info['gemm_view']
    tiles = max(1, v['grid_m']) * max(1, v['grid_n']) * g['batch'] * max(1, v['split_k'])
    bm, bn = max(1, v['block_m']), max(1, v['block_n'])
    wtm, wtn = bm / max(1, v['wave_m']), bn / max(1, v['wave_n'])
    feats = [float(v[k]) for k in KNOBS + DERIVED]
    feats += [tiles / CUS, math.ceil(tiles / CUS) * CUS / tiles, bm * bn / (bm + bn), wtm * wtn / (wtm + wtn),
              v['grid_m'] * bm / max(1, g['M']), v['grid_n'] * bn / max(1, g['N']),
              -math.log(analytic_seconds(info, v))]
    return feats


def view_of_values(info, values):
    """``info`` with the GEMM view of the task the point was solved for (a record of another task of the same
    operator carries that task's padded extents: cover - waste of each tiled axis; the batch is taken as equal)."""
    stage = info['stage_name']
    es = 2 if info['kind'] == 'f16' else 1
    ext = {ax: _get(values, stage, ax + '_cover', False) - _get(values, stage, ax + '_waste', False)
           for ax in ('grid_m', 'grid_n', 'k')}
    if min(ext.values()) <= 0:
        return info
    out = dict(info)
    out['gemm_view'] = dict(info['gemm_view'], M=ext['grid_m'], N=ext['grid_n'], K=ext['k'] // es)
    return out


def prior_score(info, values):
    """ln(1 / estimated seconds): comparable to the measured ``perf`` of a sample."""
    return featurize(info, values)[-1]


def coupled_moves(names, values, candidates):
    """Knob assignments a few coordinated steps away from ``values`` that no one-knob change reaches, for the search's
    refinement rounds: (a) the other MFMA edge at the same block tile (tile counts rescaled), (b) another number of
    K bytes per LDS row with every stage count (what fits is decided by the constraint system), each with every LDS
    swizzle, since the conflict-free swizzle depends on both, (c) the other issue order with every load spread.  ``names``: the task's knob names; ``values``: knob name ->
    value of the incumbent; ``candidates(name)``: that knob's value list.  Returns (label, knob dictionary) pairs; moves
    with the same label differ only in the dependent choices (stages, swizzle)."""
    by = {}
    for n in names:
        for k in KNOBS:
            if n.endswith("PA:" + k) or n.endswith(":" + k):
                by[k] = n
    need = ('mfma', 'tile_m', 'tile_n', 'block_k_bytes', 'lds_stages', 'lds_swizzle')
    if any(k not in by for k in need):
        return []
    out = []
    swizzles = list(candidates(by['lds_swizzle']))
    mfma, tm, tn = values[by['mfma']], values[by['tile_m']], values[by['tile_n']]
    for other in candidates(by['mfma']):
        if other == mfma or (tm * mfma) % other or (tn * mfma) % other:
            continue
        for swz in swizzles:
            out.append(("mfma=%d" % other, dict(values, **{by['mfma']: other, by['tile_m']: tm * mfma // other,
                                                           by['tile_n']: tn * mfma // other, by['lds_swizzle']: swz})))
    # (c) the other issue order with every load spread: the spread only acts on the pinned order, so a point found
    # under the compiler's order carries an arbitrary one
    if 'issue_order' in by and 'load_spread' in by:
        for order in candidates(by['issue_order']):
            if order == values[by['issue_order']]:
                continue
            for spread in candidates(by['load_spread']):
                out.append(("issue_order=%d,load_spread=%d" % (order, spread),
                            dict(values, **{by['issue_order']: order, by['load_spread']: spread})))
    for bkb in candidates(by['block_k_bytes']):
        if bkb == values[by['block_k_bytes']]:
            continue
        for stages in candidates(by['lds_stages']):
            for swz in swizzles:
                out.append(("block_k_bytes=%d" % bkb,
                            dict(values, **{by['block_k_bytes']: bkb, by['lds_stages']: stages, by['lds_swizzle']: swz})))
    return out
