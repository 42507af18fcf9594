"""Operand adapters on the CPU: pre-stage -> (oracle product in place of the kernel) -> post-stage must equal the
restatement of the reference declaration.  This checks the layout/padding logic of ``hostops.ADAPTERS`` and the
GEMM / conv views the operator definitions announce, without a GPU; the kernel itself is covered by the GPU tests.
"""
import numpy as np
import pytest
import torch

import oracle
from heron_amd import hostops
from heron_amd.ops.rocm import getOpFromName


class Ctx:
    def set_info(self, info):
        self.info = info

    def set_axis_map(self, m):
        self.axis_map = m


def rnd(shape, seed):
    return np.random.default_rng(seed).normal(0, 1, shape).astype(np.float16)


def through_adapter(name, args, inputs):
    c = Ctx()
    out = getOpFromName(name)(c, *args, "float16", "float16")
    info = c.info
    act, const, fin = hostops.ADAPTERS[info['adapter']]
    tensors = [torch.from_numpy(np.ascontiguousarray(x)) for x in inputs]
    A, Bm = act(info, *tensors), const(info, *tensors)
    assert torch.equal(Bm, hostops.prepare_constant(info, tensors))
    g = info['gemm_view']
    if info['operator'] == 'conv2d_nhwc':
        cv = info['conv']
        assert tuple(A.shape) == (cv['N'], cv['H'], cv['W'], cv['CI']) and tuple(Bm.shape) == (cv['CO'], cv['KH'], cv['KW'], cv['CI'])
        C = oracle.conv2d_nhwc_f32(A.numpy(), Bm.numpy(), (cv['stride'], cv['stride_w']), (cv['pad'], cv['pad_w']),
                                   (cv['dil'], cv['dil_w']))
        assert C.shape == out[0].shape and C.shape[0] * C.shape[1] * C.shape[2] == g['M']
    else:
        assert tuple(A.shape) == (g['M'], g['K']) and tuple(Bm.shape) == (g['N'], g['K'])
        C = oracle.gemm_f32(A.numpy(), Bm.numpy())
    assert A.is_contiguous() and Bm.is_contiguous()
    return fin(info, torch.from_numpy(C)).numpy()


def close(got, ref):
    assert got.shape == ref.shape
    assert np.abs(got - ref).max() <= 1e-4 * (np.abs(ref).max() + 1)


def test_reductions():
    A, b = rnd((33, 100), 1), rnd((1, 100), 2)
    close(through_adapter("gemv", [33, 100], [A, b]), oracle.gemv_ref(A, b))
    close(through_adapter("scan", [33, 40, 100], [A]), oracle.scan_ref(A, 40))
    In = rnd((3, 20, 7, 9), 3)
    close(through_adapter("mean", [3, 20, 7, 9], [In]), oracle.mean_ref(In))
    Mean = np.broadcast_to(In.astype(np.float64).mean(axis=(0, 2, 3), keepdims=True), In.shape).astype(np.float16)
    close(through_adapter("var", [3, 20, 7, 9], [In, Mean]), oracle.var_ref(In, Mean))


@pytest.mark.parametrize("s,p,d", [(1, 1, 1), (2, 2, 1), (1, 2, 2)])
def test_conv1d(s, p, d):
    X, F = rnd((3, 57, 12), 4), rnd((5, 12, 20), 5)
    close(through_adapter("c1d_nwc", [3, 57, 12, 20, 5, s, p, d], [X, F]), oracle.conv1d_nwc_ref(X, F, s, p, d))
    Xc, Fc = X.transpose(0, 2, 1), F.transpose(2, 1, 0)
    close(through_adapter("c1d", [3, 57, 12, 20, 5, s, p, d], [Xc, Fc]), oracle.conv1d_ncw_ref(Xc, Fc, s, p, d))


def test_conv2d_variants():
    X, F = rnd((2, 3, 20, 20), 6), rnd((16, 3, 7, 7), 7)
    close(through_adapter("c2d_nchw", [2, 20, 20, 3, 16, 7, 7, 2, 3, 1], [X, F]), oracle.conv2d_nchw_ref(X, F, 2, 3, 1))
    X, F = rnd((1, 16, 12, 15), 8), rnd((24, 16, 3, 5), 9)
    close(through_adapter("c2d_nchw", [1, 12, 15, 16, 24, 3, 5, (2, 1), (1, 2), 1], [X, F]),
          oracle.conv2d_nchw_ref(X, F, (2, 1), (1, 2), 1))
    X, F = rnd((1, 17, 13, 8), 10), rnd((3, 3, 8, 12), 11)
    close(through_adapter("dil", [1, 17, 13, 8, 12, 3, 3, 2, 3, 3], [X, F]), oracle.dil_nhwc_ref(X, F, 2, 3, 3))
    # channels-last conv with 3 input channels (the stem of the vision networks): padded to a whole chunk, no reorder
    X, F = rnd((2, 20, 20, 3), 16), rnd((16, 7, 7, 3), 17)
    close(through_adapter("c2d", [2, 20, 20, 3, 16, 7, 7, 2, 3, 1], [X, F]), oracle.conv2d_nhwc_f32(X, F, 2, 3, 1))


@pytest.mark.parametrize("s,p,d,op", [(2, 1, 1, 0), (2, 1, 1, 1), (1, 0, 1, 0), (3, 2, 2, 1)])
def test_conv2d_transposed(s, p, d, op):
    X, F = rnd((2, 6, 5, 6), 12), rnd((4, 6, 3, 4), 13)
    close(through_adapter("t2d", [2, 5, 6, 6, 4, 3, 4, s, p, d, op], [X, F]), oracle.conv2d_transposed_nchw_ref(X, F, s, p, d, op))


@pytest.mark.parametrize("s,p,d", [(1, 1, 1), ((2, 1, 1), (1, 1, 0), 1), (1, (0, 2, 1), (2, 2, 1))])
def test_conv3d(s, p, d):
    X, F = rnd((2, 6, 9, 7, 5), 14), rnd((3, 3, 2, 5, 12), 15)
    close(through_adapter("c3d_ndhwc", [2, 6, 9, 7, 5, 12, 3, 3, 2, s, p, d], [X, F]), oracle.conv3d_ndhwc_ref(X, F, s, p, d))
    Xc, Fc = X.transpose(0, 4, 1, 2, 3), F.transpose(4, 3, 0, 1, 2)
    close(through_adapter("c3d", [2, 6, 9, 7, 5, 12, 3, 3, 2, s, p, d], [Xc, Fc]), oracle.conv3d_ncdhw_ref(Xc, Fc, s, p, d))


@pytest.mark.parametrize("s,p,mult", [(1, 1, 1), (2, 1, 2)])
def test_depthwise(s, p, mult):
    X, F = rnd((2, 6, 9, 8), 16), rnd((6 * mult, 3, 3), 17)
    c = Ctx()
    out = getOpFromName("dep")(c, 2, 9, 8, 6, 6 * mult, 3, 3, s, p, 1, "float16", "float16")
    act, const, fin = hostops.ADAPTERS[c.info['adapter']]
    A, Bm = act(c.info, torch.from_numpy(X), torch.from_numpy(F)), const(c.info, torch.from_numpy(X), torch.from_numpy(F))
    g = c.info['gemm_view']
    assert tuple(A.shape) == (g['batch'], g['M'], g['K']) and tuple(Bm.shape) == (g['batch'], g['N'], g['K'])
    C = oracle.bmm_f32(A.numpy(), Bm.numpy())
    close(fin(c.info, torch.from_numpy(C)).numpy(), oracle.depthwise_conv2d_ref(X, F, s, p))


# ---------------------------------------------------------------------------------------------------------------
# The index maps the adapters hand to the library's gather pass (hrn_gather_nd), evaluated here by a plain loop over
# the destination index space: with device tensors the adapters build these maps instead of calling torch, so the
# maps must yield what the torch formulation of the same pre-stage yields.
def emulate_gather(src, out, dst_dim, coords, dst_stride=None, dst_live=None, op=0, aux=None):
    import itertools
    s_flat, o_flat = src.reshape(-1).numpy(), out.reshape(-1).numpy()
    a_flat = aux.reshape(-1).numpy() if aux is not None else None
    nd = len(dst_dim)
    if dst_stride is None:
        dst_stride = [int(np.prod(dst_dim[d + 1:])) for d in range(nd)]
    live_ext = dst_live if dst_live is not None else dst_dim
    assert dst_stride[-1] == 1
    for idx in itertools.product(*[range(int(e)) for e in dst_dim]):
        doff = sum(i * st for i, st in zip(idx, dst_stride))
        live = all(i < l for i, l in zip(idx, live_ext))
        soff = 0
        for entry in coords:
            extent, stride, muls = entry[0], entry[1], entry[2]
            add = entry[3] if len(entry) > 3 else 0
            div = entry[4] if len(entry) > 4 else 1
            num = add + sum(m * idx[d] for d, m in muls.items())
            if num < 0 or num % div or num // div >= extent:
                live = False
            soff += (num // div) * stride
        if not live:
            o_flat[doff] = 0
        elif op == 0:
            o_flat[doff] = s_flat[soff]
        else:
            d = np.float16(s_flat[soff] - a_flat[soff])
            o_flat[doff] = np.float16(d * d)
    return out


def both_paths(monkeypatch, fn, info, *tensors):
    """The adapter half ``fn`` through its torch formulation and through the emulated library passes."""
    via_torch = fn(info, *tensors)
    with monkeypatch.context() as m:
        m.setattr(hostops, "_native_ok", lambda t: True)
        m.setattr(hostops, "_gather", emulate_gather)
        m.setattr(hostops, "_channels_last", lambda x3, cp=None: hostops._pad_last(x3.permute(0, 2, 1), cp or x3.shape[1]))
        via_maps = fn(info, *tensors)
    assert via_maps.shape == via_torch.shape and via_maps.is_contiguous()
    assert torch.equal(via_maps, via_torch)


def info_of(name, args):
    c = Ctx()
    getOpFromName(name)(c, *args, "float16", "float16")
    return c.info


def test_gather_maps_equal_the_torch_formulation(monkeypatch):
    t = lambda shape, seed: torch.from_numpy(rnd(shape, seed))
    In = t((3, 10, 4, 6), 20)
    both_paths(monkeypatch, hostops._act_mean, info_of("mean", [3, 10, 4, 6]), In)
    both_paths(monkeypatch, hostops._act_var, info_of("var", [3, 10, 4, 6]), In, t((3, 10, 4, 6), 21))
    In = t((1, 5, 3, 3), 22)                                    # N*H*W = 9: the rows of A are padded to 16
    both_paths(monkeypatch, hostops._act_mean, info_of("mean", [1, 5, 3, 3]), In)
    for s, p, d in [(1, 1, 1), ((2, 1, 1), (1, 1, 0), 1), (1, (0, 2, 1), (2, 2, 1))]:
        X, F = t((2, 6, 5, 4, 5), 23), t((3, 3, 2, 5, 12), 24)
        both_paths(monkeypatch, hostops._act_c3d_ndhwc, info_of("c3d_ndhwc", [2, 6, 5, 4, 5, 12, 3, 3, 2, s, p, d]), X, F)
    for s, p, d, op in [(2, 1, 1, 0), (2, 1, 1, 1), (1, 0, 1, 0), (3, 2, 2, 1)]:
        X, F = t((2, 6, 5, 6), 25), t((4, 6, 3, 4), 26)
        both_paths(monkeypatch, hostops._act_t2d_nchw, info_of("t2d", [2, 5, 6, 6, 4, 3, 4, s, p, d, op]), X, F)
    for s, p, mult in [(1, 1, 1), (2, 1, 2)]:
        X, F = t((2, 6, 9, 8), 27), t((6 * mult, 3, 3), 28)
        info = info_of("dep", [2, 9, 8, 6, 6 * mult, 3, 3, s, p, 1])
        both_paths(monkeypatch, hostops._act_dep, info, X, F)
        g = info['gemm_view']
        both_paths(monkeypatch, hostops._fin_dep, info, t((g['batch'], g['M'], g['N']), 29))
