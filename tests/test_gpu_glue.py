"""GPU parity of the glue operators against closed forms / the oracle (the reference CPU
backend where built).  Tolerances are the per-op NMSE limits of tests/test-backend-ops.cpp
(:319 default 1e-7, :2375 soft_max 1e-6, :1451 cpy 1e-6)."""
import ctypes as C

import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu


def _t(dev, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _d(t):
    import mi355
    return C.byref(mi355.tensor_desc(t))


@pytest.mark.parametrize("ncols,nrows", [(4096, 7), (64, 5), (1, 3), (14336, 2)])
def test_rms_norm(dev, ncols, nrows):
    import torch
    import mi355
    rng = np.random.default_rng(1)
    x = rng.standard_normal((nrows, ncols)).astype(np.float32)
    xd = _t(dev, x)
    yd = torch.empty_like(xd)
    mi355.check(mi355.load().mi355_rms_norm(None, _d(xd), _d(yd), 1e-5))
    want = np.zeros_like(x)
    orc.oracle.orc_rms_norm(orc._ptr(x), orc._ptr(want), ncols, nrows, 1e-5)
    assert orc.nmse(yd.cpu().numpy(), want) < 1e-7
    # strided rows (a view taking every other row)
    big = _t(dev, np.repeat(x, 2, axis=0))
    view = big[::2]
    mi355.check(mi355.load().mi355_rms_norm(None, _d(view), _d(yd), 1e-5))
    assert orc.nmse(yd.cpu().numpy(), want) < 1e-7


@pytest.mark.parametrize("op,fn", [(0, np.add), (1, np.subtract), (2, np.multiply), (3, np.divide)])
@pytest.mark.parametrize("sa,sb", [((5, 4096), (1, 4096)), ((3, 2, 64), (3, 2, 1)), ((6, 4), (6, 1)), ((2, 3, 4, 8), (1, 3, 1, 8)),
                                   ((7, 33), (7, 33))])
def test_bin_bcast(dev, op, fn, sa, sb):
    import torch
    import mi355
    rng = np.random.default_rng(2)
    a = rng.standard_normal(sa).astype(np.float32)
    b = (rng.standard_normal(sb).astype(np.float32) + 3.0)
    ad, bd = _t(dev, a), _t(dev, b)
    od = torch.empty_like(ad)
    mi355.check(mi355.load().mi355_bin_bcast(None, op, _d(ad), _d(bd), _d(od)))
    assert orc.nmse(od.cpu().numpy(), fn(a, b)) < 1e-7


def test_add_row_strided_views(dev):
    """the MoE combine adds two row-strided views of one [N, 2, T] tensor"""
    import torch
    import mi355
    rng = np.random.default_rng(3)
    e = rng.standard_normal((9, 2, 128)).astype(np.float32)
    ed = _t(dev, e)
    a, b = ed[:, 0, :], ed[:, 1, :]
    od = torch.empty((9, 128), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_bin_bcast(None, 0, _d(a), _d(b), _d(od)))
    assert np.array_equal(od.cpu().numpy(), e[:, 0] + e[:, 1])


def test_unary_and_scale(dev):
    import torch
    import mi355
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((3, 14336)) * 4).astype(np.float32)
    xd = _t(dev, x)
    yd = torch.empty_like(xd)
    lib = mi355.load()
    mi355.check(lib.mi355_unary(None, 10, _d(xd), _d(yd)))
    want = np.zeros_like(x)
    orc.oracle.orc_silu(orc._ptr(x), orc._ptr(want), x.size)
    assert orc.nmse(yd.cpu().numpy(), want) < 1e-7
    x64 = x.astype(np.float64)
    for op, ref in [(0, np.abs(x64)), (2, -x64), (4, np.tanh(x64)), (6, np.maximum(x64, 0)), (7, 1 / (1 + np.exp(-x64))),
                    (13, np.exp(x64)), (8, 0.5 * x64 * (1 + np.tanh(0.7978845608028654 * x64 * (1 + 0.044715 * x64 * x64))))]:
        mi355.check(lib.mi355_unary(None, op, _d(xd), _d(yd)))
        assert orc.nmse(yd.cpu().numpy(), ref) < 1e-7, op
    mi355.check(lib.mi355_scale(None, _d(xd), _d(yd), 0.125))
    assert np.array_equal(yd.cpu().numpy(), x * np.float32(0.125))


def test_cpy_types_and_strides(dev):
    import torch
    import mi355
    rng = np.random.default_rng(5)
    lib = mi355.load()
    x = rng.standard_normal((5, 8, 128)).astype(np.float32)
    xd = _t(dev, x)
    # f32 -> f16 (KV cache write): round to nearest even like GGML_FP32_TO_FP16
    hd = torch.empty((5, 8, 128), dtype=torch.float16, device=dev)
    mi355.check(lib.mi355_cpy(None, _d(xd), _d(hd)))
    want = np.zeros(x.size, dtype=np.uint16)
    orc.oracle.orc_f32_to_f16_row(orc._ptr(x), orc._ptr(want), x.size)
    assert np.array_equal(hd.cpu().numpy().view(np.uint16).ravel(), want)
    # permuted source -> contiguous destination (CONT), different shape with equal element count
    pd = xd.permute(1, 0, 2)
    cd = torch.empty((8, 5 * 128), dtype=torch.float32, device=dev)
    mi355.check(lib.mi355_cpy(None, _d(pd), _d(cd)))
    assert np.array_equal(cd.cpu().numpy(), x.transpose(1, 0, 2).reshape(8, -1))
    # f16 -> f32 and into a strided destination view
    big = torch.zeros((5, 8, 256), dtype=torch.float32, device=dev)
    mi355.check(lib.mi355_cpy(None, _d(hd), _d(big[:, :, 64:192])))
    assert np.array_equal(big.cpu().numpy()[:, :, 64:192], hd.cpu().numpy().astype(np.float32))
    assert (big.cpu().numpy()[:, :, :64] == 0).all()


def test_get_rows(dev):
    import torch
    import mi355
    rng = np.random.default_rng(6)
    src = rng.standard_normal((50, 4096)).astype(np.float32)
    ids = rng.integers(0, 50, 17).astype(np.int32)
    sd, idd = _t(dev, src), _t(dev, ids)
    od = torch.empty((17, 4096), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_get_rows(None, _d(sd), _d(idd), _d(od)))
    assert np.array_equal(od.cpu().numpy(), src[ids])
    # MoE: src [T, 8, 1] gathered by ids [T, 2] taken as a strided view of [T, 8]
    T = 12
    w = rng.standard_normal((T, 8, 1)).astype(np.float32)
    full = np.stack([rng.permutation(8) for _ in range(T)]).astype(np.int32)
    wd, fd = _t(dev, w), _t(dev, full)
    sel = fd[:, :2]
    od = torch.empty((T, 2, 1), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_get_rows(None, _d(wd), _d(sel), _d(od)))
    want = np.stack([w[t, full[t, :2], :] for t in range(T)])
    assert np.array_equal(od.cpu().numpy(), want)


@pytest.mark.parametrize("name,t", list(orc.WEIGHT_TYPES.items()))
@pytest.mark.parametrize("K", [256, 4096])
def test_get_rows_quantized(dev, name, t, K):
    """rows of a quantized matrix held in the device layout come back as dequantize_row_* of the original blocks, bit for bit
    against the oracle's restatement (one product and one difference per element, no sums to reorder)"""
    import ctypes as C
    import torch
    import mi355
    rng = np.random.default_rng(K + t)
    n_rows, n_get = 40, 23
    raw = orc.quantize("oracle", t, (rng.standard_normal((n_rows, K)) * 0.1).astype(np.float32))
    W = mi355.upload_weights(t, _t(dev, raw))
    ids = rng.integers(0, n_rows, n_get).astype(np.int32)
    idd = _t(dev, ids)
    od = torch.zeros((n_get, K), dtype=torch.float32, device=dev)
    src = mi355.Tensor()
    src.data, src.type = W.data_ptr(), t
    rb = raw.shape[1]
    for i, (ne, nb) in enumerate(((K, rb // (K // mi355.BLOCK[t][0])), (n_rows, rb), (1, rb * n_rows), (1, rb * n_rows))):
        src.ne[i], src.nb[i] = ne, nb
    mi355.check(mi355.load().mi355_get_rows(None, C.byref(src), _d(idd), _d(od)))
    want = orc.dequantize("oracle", t, raw, K)[ids]
    got = od.cpu().numpy()
    if t in (orc.Q4_0, orc.Q8_0, orc.Q6_K, orc.Q5_0, orc.IQ4_NL, orc.IQ4_XS):
        assert np.array_equal(got, want)                      # a single product chain per element
    else:
        assert np.max(np.abs(got - want)) <= 1e-6 * np.max(np.abs(want))   # d*sc*n - dmin*m: the compiler may fuse the subtraction


@pytest.mark.parametrize("ncols,nrows,masked", [(8, 512, False), (1024, 6, True), (33, 5, True)])
def test_soft_max(dev, ncols, nrows, masked):
    import torch
    import mi355
    rng = np.random.default_rng(7)
    x = rng.standard_normal((nrows, ncols)).astype(np.float32) * 3
    m = rng.standard_normal((nrows, ncols)).astype(np.float32) if masked else None
    xd = _t(dev, x)
    od = torch.empty_like(xd)
    md = _t(dev, m) if masked else None
    mi355.check(mi355.load().mi355_soft_max(None, _d(xd), _d(md) if masked else None, _d(od), 0.7, 0.0))
    want = np.zeros_like(x)
    orc.oracle.orc_soft_max(orc._ptr(x), orc._ptr(m), orc._ptr(want), ncols, nrows, 0.7)
    assert orc.nmse(od.cpu().numpy(), want) < 1e-6
    if masked:   # f16 mask
        mh = m.astype(np.float16)
        mi355.check(mi355.load().mi355_soft_max(None, _d(xd), _d(_t(dev, mh)), _d(od), 0.7, 0.0))
        mf = mh.astype(np.float32)
        orc.oracle.orc_soft_max(orc._ptr(x), orc._ptr(mf), orc._ptr(want), ncols, nrows, 0.7)
        assert orc.nmse(od.cpu().numpy(), want) < 1e-6


@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("n_dims,ne0", [(128, 128), (64, 128)])
@pytest.mark.parametrize("ff,ext", [(False, 0.0), (True, 0.0), (False, 1.0)])
def test_rope(dev, mode, n_dims, ne0, ff, ext):
    import torch
    import mi355
    rng = np.random.default_rng(8)
    heads, T = 8, 9
    x = rng.standard_normal((T, heads, ne0)).astype(np.float32)
    pos = rng.integers(0, 4096, T).astype(np.int32)
    fac = (1.0 + rng.uniform(0, 1, n_dims // 2)).astype(np.float32) if ff else None
    fs = 0.5 if ext else 1.0
    xd, pd = _t(dev, x), _t(dev, pos)
    fd = _t(dev, fac) if ff else None
    od = torch.empty_like(xd)
    mi355.check(mi355.load().mi355_rope(None, _d(xd), pd.data_ptr(), fd.data_ptr() if ff else None, _d(od), n_dims, mode, 8192,
                                        500000.0, fs, ext, 1.0, 32.0, 1.0))
    want = np.zeros_like(x)
    orc.oracle.orc_rope(orc._ptr(x), orc._ptr(pos), orc._ptr(fac), orc._ptr(want), ne0, heads, T, n_dims, mode, 500000.0, fs,
                        ext, 1.0, 32.0, 1.0, 8192)
    assert orc.nmse(od.cpu().numpy(), want) < 1e-7


def test_sum_rows_argsort(dev):
    import torch
    import mi355
    rng = np.random.default_rng(9)
    lib = mi355.load()
    x = rng.standard_normal((37, 8)).astype(np.float32)
    xd = _t(dev, x)
    sd = torch.empty((37, 1), dtype=torch.float32, device=dev)
    mi355.check(lib.mi355_sum_rows(None, _d(xd), _d(sd)))
    assert orc.nmse(sd.cpu().numpy().ravel(), x.astype(np.float64).sum(1)) < 1e-7
    for ncols in (8, 16, 100, 1024):
        v = np.stack([rng.permutation(ncols) for _ in range(5)]).astype(np.float32)   # distinct values: order is unambiguous
        vd = _t(dev, v)
        for order in (0, 1):
            idd = torch.empty((5, ncols), dtype=torch.int32, device=dev)
            mi355.check(lib.mi355_argsort(None, _d(vd), _d(idd), order))
            want = np.zeros((5, ncols), dtype=np.int32)
            orc.oracle.orc_argsort(orc._ptr(v), orc._ptr(want), ncols, 5, order)
            assert np.array_equal(idd.cpu().numpy(), want)


def test_mul_mat_f(dev):
    import torch
    import mi355
    rng = np.random.default_rng(10)
    W = rng.standard_normal((8, 4096)).astype(np.float32)
    x = rng.standard_normal((33, 4096)).astype(np.float32)
    wd, xd = _t(dev, W), _t(dev, x)
    od = torch.empty((33, 8), dtype=torch.float32, device=dev)
    mi355.check(mi355.load().mi355_mul_mat_f(None, _d(wd), _d(xd), _d(od)))
    assert orc.nmse(od.cpu().numpy(), x.astype(np.float64) @ W.astype(np.float64).T) < 1e-7
    wh = _t(dev, W.astype(np.float16))
    mi355.check(mi355.load().mi355_mul_mat_f(None, _d(wh), _d(xd), _d(od)))
    assert orc.nmse(od.cpu().numpy(), x.astype(np.float64) @ W.astype(np.float16).astype(np.float64).T) < 1e-7
