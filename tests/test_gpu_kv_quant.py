"""GPU parity of the quantized KV cache path: CPY f32 -> Q8_0 / Q4_0 (bit-exact with the reference quantizers) and FLASH_ATTN_EXT over
Q8_0 / Q4_0 K and V against the oracle's restatement of the reference CPU kernel, the reference CPU backend itself and the textbook
form on the dequantized cache."""
import numpy as np
import pytest

import orc

pytestmark = pytest.mark.gpu

KV_TYPES = [("f16", orc.F16), ("q8_0", orc.Q8_0), ("q4_0", orc.Q4_0)]


def _special(rng, n_rows, k):
    x = rng.standard_normal((n_rows, k)).astype(np.float32)
    x[0, :32] = 0.0                                   # an all-zero block
    x[1, :32] = 0.0
    x[1, 7] = -3.0                                    # a single extreme
    x[2, :32] = np.linspace(-127.5, 127.5, 32) / 127.0 * 4.0   # levels that land on .5 ties for Q8_0
    x[3, :32] = np.where(np.arange(32) % 2 == 0, 2.0, -2.0)    # +max and -max of equal magnitude: the first one sets the sign (Q4_0)
    x[4, :32] = -x[3, :32]
    return x


@pytest.mark.parametrize("name,t", KV_TYPES[1:])
@pytest.mark.parametrize("rows,k", [(8, 128), (40, 1024), (5, 32)])
def test_cpy_f32_quant_bit_exact(dev, name, t, rows, k):
    """plain ggml block placement and the device row layout (with an offset of whole rows, as a cache store at cell kv_head has)"""
    import torch
    import mi355
    lib = mi355.load()
    rng = np.random.default_rng(rows + k + t)
    x = _special(rng, rows, k)
    want = orc.quantize("ref" if orc.ref is not None else "oracle", t, x)
    assert np.array_equal(want, orc.quantize("oracle", t, x))
    xd = torch.from_numpy(x).to(dev)
    plain = torch.zeros(want.shape, dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_cpy_f32_quant(None, t, xd.data_ptr(), plain.data_ptr(), 0, 0, rows * k))
    torch.cuda.synchronize()
    assert np.array_equal(plain.cpu().numpy(), want)
    # a "cache" of rows + 3 rows in the device layout; the store starts at row 3
    nb = k // 32
    cache = torch.zeros((rows + 3, want.shape[1]), dtype=torch.uint8, device=dev)
    mi355.check(lib.mi355_cpy_f32_quant(None, t, xd.data_ptr(), cache.data_ptr(), 3 * nb, nb, rows * k))
    torch.cuda.synchronize()
    back = mi355.download_weights(t, cache).cpu().numpy()
    assert np.array_equal(back[3:], want)
    assert not back[:3].any()


def _case(rng, D, Nq, Nkv, Hq, Hkv):
    q = rng.standard_normal((Hq, Nq, D)).astype(np.float32)
    kf = rng.standard_normal((Hkv, Nkv, D)).astype(np.float32)
    vf = rng.standard_normal((Hkv, Nkv, D)).astype(np.float32)
    nq_pad = (Nq + 63) // 64 * 64
    j = np.arange(Nkv)[None, :]
    i = np.arange(nq_pad)[:, None]
    mask = np.where(j <= Nkv - Nq + i, 0.0, -np.inf).astype(np.float32)
    mask[Nq:] = -np.inf
    mask = (mask + np.where(np.isfinite(mask), rng.uniform(-1, 1, mask.shape), 0.0)).astype(np.float16)
    return q, kf, vf, mask


def _textbook(q, k, tk, v, tv, mask, scale, q_as_q8_0=False):
    """q_as_q8_0: q rounded to Q8_0 first, as ggml-cpu does for a quantized K (its dot is the integer block dot, ggml-cpu.c:11037-11046)"""
    Hq, Nq, D = q.shape
    if q_as_q8_0:
        q = orc.dequantize("oracle", orc.Q8_0, orc.quantize("oracle", orc.Q8_0, q.reshape(Hq * Nq, D)), D).reshape(Hq, Nq, D)
    Hkv, Nkv = k.shape[0], k.shape[1]

    def deq(a, t):
        if t == orc.F16:
            return a.view(np.float16).astype(np.float64).reshape(Hkv, Nkv, D)
        return orc.dequantize("oracle", t, a.reshape(Hkv * Nkv, -1), D).reshape(Hkv, Nkv, D).astype(np.float64)
    kd, vd = deq(k, tk), deq(v, tv)
    rep = Hq // Hkv
    out = np.zeros((Nq, Hq, D))
    for h in range(Hq):
        s = q[h].astype(np.float64) @ kd[h // rep].T * scale + mask[:Nq].astype(np.float64)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (p / p.sum(axis=1, keepdims=True)) @ vd[h // rep]
    return out


def _run(dev, q, k, tk, v, tv, mask, scale, device_layout):
    """k, v: uint8 [Hkv, Nkv, row bytes] in ggml block layout.  device_layout: True - the cache is a [cells][Hkv * D] tensor kept in the
    device row layout, addressed through its rows; "1d" - a 1-D tensor of all cells in the device row layout (what a llama.cpp cache
    tensor in a plug-in buffer is: src/llama-kv-cache.cpp:94-95 allocates them with ggml_new_tensor_1d)"""
    import torch
    import mi355
    lib = mi355.load()
    Hq, Nq, D = q.shape
    Hkv, Nkv = k.shape[0], k.shape[1]
    qd = torch.from_numpy(q).to(dev)
    md = torch.from_numpy(mask).to(dev)
    dst = torch.empty((Nq, Hq, D), dtype=torch.float32, device=dev)

    def operand(a, t):
        rb = a.shape[2]
        if t == orc.F16:   # [cell][head][D] like the cache
            d = torch.from_numpy(np.ascontiguousarray(a.transpose(1, 0, 2))).to(dev)
            return d, d.data_ptr(), None, 0, Hkv * rb, rb
        if not device_layout:   # plain blocks, [head][cell] rows
            d = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
            return d, d.data_ptr(), None, 0, rb, Nkv * rb
        cells = np.ascontiguousarray(a.transpose(1, 0, 2)).reshape(Nkv, Hkv * rb)     # one row of Hkv * D elements per cell
        if device_layout == "1d":   # llama.cpp's cache tensors are 1-D: ONE row of all cells (all levels first, all scales behind them)
            d = mi355.upload_weights(t, torch.from_numpy(cells.reshape(1, -1)).to(dev))
            return d, d.data_ptr(), d.data_ptr(), Nkv * Hkv * D // 32, Hkv * rb, rb
        d = mi355.upload_weights(t, torch.from_numpy(cells).to(dev))
        return d, d.data_ptr(), d.data_ptr(), Hkv * D // 32, Hkv * rb, rb
    kd, kp, kbase, krb, k_nb1, k_nb2 = operand(k, tk)
    vd, vp, vbase, vrb, v_nb1, v_nb2 = operand(v, tv)
    need = int(lib.mi355_flash_attn_kv_ws_bytes(D, Nq, Nkv, Hq, Hkv, tk, tv))
    ws = torch.empty(need + 256, dtype=torch.uint8, device=dev)
    wp = (ws.data_ptr() + 255) & ~255
    mi355.check(lib.mi355_flash_attn_ext_kv(None, qd.data_ptr(), kp, tk, kbase, krb, vp, tv, vbase, vrb, md.data_ptr(), dst.data_ptr(), D, Nq, Nkv, Hq, Hkv,
                                            D * 4, Nq * D * 4, k_nb1, k_nb2, v_nb1, v_nb2, mask.shape[1] * 2, scale, 0.0, 0.0, wp, need, None))
    torch.cuda.synchronize()
    return dst.cpu().numpy()


@pytest.mark.parametrize("name,t", KV_TYPES[1:])
@pytest.mark.parametrize("src_rb,dst_rb", [(0, 0), (0, 8), (8, 0), (8, 8), (72, 72)])
def test_cpy_quant_blocks(dev, name, t, src_rb, dst_rb):
    """ranges of blocks copied between two quantized tensors (the row copies of a cache defragmentation), each side in plain ggml
    block order or in the device row layout with 8 blocks per row / as one row of 72 blocks"""
    import torch
    import mi355
    lib = mi355.load()
    rng = np.random.default_rng(t + src_rb + 3 * dst_rb)
    nb = 72
    a = orc.quantize("oracle", t, _special(rng, 9, 256))      # 72 blocks
    b = orc.quantize("oracle", t, _special(rng, 9, 256))

    def up(x, rb):
        if rb == 0:
            return torch.from_numpy(x).to(dev)
        return mi355.upload_weights(t, torch.from_numpy(x.reshape(nb // rb, -1)).to(dev))

    def down(d, rb):
        return (d if rb == 0 else mi355.download_weights(t, d)).cpu().numpy().reshape(-1)
    ad, bd = up(a, src_rb), up(b, dst_rb)
    bb = a.size // nb
    mi355.check(lib.mi355_cpy_quant_blocks(None, t, ad.data_ptr(), 37, src_rb, bd.data_ptr(), 5, dst_rb, 29))
    torch.cuda.synchronize()
    want = b.reshape(-1).copy()
    want[5 * bb:(5 + 29) * bb] = a.reshape(-1)[37 * bb:(37 + 29) * bb]
    assert np.array_equal(down(bd, dst_rb), want)
    assert np.array_equal(down(ad, src_rb), a.reshape(-1))


@pytest.mark.parametrize("name,t", KV_TYPES[1:])
@pytest.mark.parametrize("device_layout", [False, True])
def test_cpy_quant_view_both_directions(dev, name, t, device_layout):
    """the two copies around the ROPE of a quantized cache's K-shift (build_k_shift, src/llama.cpp:1167-1213): a [D, heads, cells] view of
    the cache cast to f32, and contiguous f32 rows copied back into such a view - here a view that skips cells and takes every second
    head, so that all three block strides matter; blocks in plain ggml order and in the device row layout"""
    import ctypes
    import torch
    import mi355
    lib = mi355.load()
    D, H, C = 64, 6, 9                       # cache: C cells of H heads of D elements
    rng = np.random.default_rng(t + 11 * device_layout)
    x = _special(rng, C, H * D)              # what the cache holds
    rows = orc.quantize("oracle", t, x)      # [C, row bytes] in ggml block order
    bb = rows.shape[1] // (H * D // 32)
    cache = mi355.upload_weights(t, torch.from_numpy(rows).to(dev)) if device_layout else torch.from_numpy(rows).to(dev)
    rb = H * D // 32 if device_layout else 0
    # the view: cells 2.., heads 1, 3, 5: element (i0, i1, i2) at cell 2 + i2, head 1 + 2 i1
    ne = (ctypes.c_int64 * 4)(D, 3, C - 2, 1)
    strides = (ctypes.c_int64 * 3)(2 * D // 32, H * D // 32, 0)
    first = (2 * H + 1) * D // 32
    f = torch.empty((C - 2, 3, D), dtype=torch.float32, device=dev)
    mi355.check(lib.mi355_cpy_quant_view(None, t, 1, f.data_ptr(), cache.data_ptr(), first, rb, ne, strides))
    torch.cuda.synchronize()
    full = orc.dequantize("oracle", t, rows, H * D).reshape(C, H, D)
    assert np.array_equal(f.cpu().numpy(), full[2:, 1::2])
    # back: new values into the same view; everything outside it keeps its bytes
    y = _special(rng, (C - 2) * 3, D)
    yd = torch.from_numpy(y).to(dev)
    mi355.check(lib.mi355_cpy_quant_view(None, t, 0, yd.data_ptr(), cache.data_ptr(), first, rb, ne, strides))
    torch.cuda.synchronize()
    got = (mi355.download_weights(t, cache) if device_layout else cache).cpu().numpy().reshape(C, H, D // 32 * bb)
    want = rows.reshape(C, H, D // 32 * bb).copy()
    want[2:, 1::2] = orc.quantize("oracle", t, y).reshape(C - 2, 3, -1)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("kname,tk", KV_TYPES)
@pytest.mark.parametrize("vname,tv", KV_TYPES)
@pytest.mark.parametrize("D,Nq,Nkv,Hq,Hkv", [(128, 1, 256, 32, 8), (128, 1, 4096, 32, 8), (128, 40, 700, 8, 2), (64, 3, 96, 6, 3)])
@pytest.mark.parametrize("device_layout", [False, True, "1d"])
def test_flash_attn_quantized_kv(dev, kname, tk, vname, tv, D, Nq, Nkv, Hq, Hkv, device_layout):
    if tk == orc.F16 and tv == orc.F16 and device_layout:
        pytest.skip("f16 rows have one layout")
    rng = np.random.default_rng(D + Nq + Nkv + tk * 3 + tv)
    q, kf, vf, mask = _case(rng, D, Nq, Nkv, Hq, Hkv)
    k, v = orc.kv_rows(tk, kf), orc.kv_rows(tv, vf)
    scale = 1.0 / np.sqrt(D)
    got = _run(dev, q, k, tk, v, tv, mask, scale, device_layout)
    assert np.isfinite(got).all()
    # exact arithmetic on the dequantized cache: only the f16 rounding of q and of d * level separates the two (the streaming kernel,
    # which one token over 1024+ cells of a fully quantized cache in the device layout takes, rounds q to Q8_0 as ggml-cpu does)
    streaming = device_layout and Nq == 1 and Nkv >= 1024 and tk != orc.F16 and tv != orc.F16
    assert orc.nmse(got, _textbook(q, k, tk, v, tv, mask, scale, q_as_q8_0=streaming)) < 1e-5
    # the reference kernel quantizes q to Q8_0 for a quantized K: its own distance from exact is ~2e-5
    if Nq * Nkv * Hq <= 40 * 700 * 8:
        assert orc.nmse(got, orc.flash_attn_kv("cpu", q, k, tk, v, tv, mask.view(np.uint16), scale)) <= 5e-4      # tests/test-backend-ops.cpp:3137
    if orc.ref is not None:
        assert orc.nmse(got, orc.flash_attn_kv("ref", q, k, tk, v, tv, mask.view(np.uint16), scale, n_threads=16)) <= 5e-4


@pytest.mark.parametrize("kname,tk", [kt for kt in KV_TYPES if kt[1] != orc.F16])
@pytest.mark.parametrize("vname,tv", [kt for kt in KV_TYPES if kt[1] != orc.F16])
@pytest.mark.parametrize("Nkv,Hq,Hkv", [(1024, 32, 8), (4096, 32, 8), (5000, 32, 8), (16421, 32, 8), (2048, 8, 8), (3000, 16, 8), (40000, 8, 2)])
@pytest.mark.parametrize("layout", [True, "1d"])
def test_flash_attn_quantized_kv_streaming(dev, kname, tk, vname, tv, Nkv, Hq, Hkv, layout):
    """one token over a long quantized cache in the device row layout: the streaming kernel (levels and scales by global-to-LDS transfers,
    integer block dots of Q8_0-quantized q with K, V expanded to f16 inside the wave).  Held to the reference's arithmetic - exact
    sums with q rounded to Q8_0 - and, more loosely, to the sums with q unrounded; ragged last tiles, one to four heads per kv head."""
    D = 128
    rng = np.random.default_rng(Nkv + Hq + tk * 3 + tv)
    q, kf, vf, mask = _case(rng, D, 1, Nkv, Hq, Hkv)
    k, v = orc.kv_rows(tk, kf), orc.kv_rows(tv, vf)
    scale = 1.0 / np.sqrt(D)
    got = _run(dev, q, k, tk, v, tv, mask, scale, layout)
    assert np.isfinite(got).all()
    assert orc.nmse(got, _textbook(q, k, tk, v, tv, mask, scale, q_as_q8_0=True)) < 1e-5
    assert orc.nmse(got, _textbook(q, k, tk, v, tv, mask, scale)) < 5e-4
    if orc.ref is not None:   # ggml-cpu itself: same rounding of q, same integer dots; its V sum runs in f16 for f16 V only
        assert orc.nmse(got, orc.flash_attn_kv("ref", q, k, tk, v, tv, mask.view(np.uint16), scale, n_threads=16)) <= 1e-5
